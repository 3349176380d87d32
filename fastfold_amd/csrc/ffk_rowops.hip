// Row-wise HBM-bound kernels: fused mask+bias softmax, LayerNorm (forward and backward)
// and the three elementwise fusions.  Rows are short (128..4096 elements), so a row is
// owned by a group of `lpr` adjacent lanes of one 64-wide wavefront (several rows per
// wave), every lane moves 16 bytes per access and consecutive lanes touch consecutive
// 16-byte vectors: each wave-level access covers whole 128-byte lines.  Reductions are
// xor-shuffles inside the lane group; all arithmetic is fp32.
#include "ffk_common.h"
#include <stdlib.h>

thread_local char ffk_err_buf[512] = "";

int ffk_fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(ffk_err_buf, sizeof(ffk_err_buf), fmt, ap);
    va_end(ap);
    return code;
}

std::mutex& ffk_config_mutex() {
    static std::mutex m;
    return m;
}

extern "C" int ffk_version(void) { return 110; }
extern "C" const char* ffk_last_error_string(void) { return ffk_err_buf; }

namespace {

constexpr int WAVES_PER_BLOCK = 4;
constexpr int BLOCK = 64 * WAVES_PER_BLOCK;
constexpr float MASK_FILL = -1e9f;

// Lane-group geometry for a row of `nvec` 16-byte vectors: lanes per row (power of two,
// 4..64) and vectors per lane (1, 2, 4 or 8).  Returns false if the row does not fit.
struct RowGeom {
    int lpr, vpl;
};
// every (lanes per row, vectors per lane) pair row_geom can return
#define FFK_ROW_GEOMETRIES(X) X(8, 1) X(8, 2) X(8, 4) X(16, 4) X(32, 4) X(64, 4) X(64, 8)
static bool row_geom(long nvec, RowGeom* g) {
    constexpr int min_lpr = 8;
    constexpr int tgt_vpl = 4;
    int lpr = min_lpr;   // >= 8 lanes x 16 B: every wave-level access covers whole 128-byte lines
    while (lpr < 64 && (long)lpr * tgt_vpl < nvec) lpr <<= 1;
    long vpl = (nvec + lpr - 1) / lpr;
    int v = 1;
    while (v < vpl) v <<= 1;
    if (v > 8) return false;
    g->lpr = lpr;
    g->vpl = v;
    return true;
}

static int row_grid(long rows, int lpr) {
    long rows_per_block = (long)WAVES_PER_BLOCK * (64 / lpr);
    long blocks = (rows + rows_per_block - 1) / rows_per_block;
    constexpr long cap = 256L * 16;   // 256 CUs x resident blocks; grid-stride beyond
    return (int)(blocks < cap ? blocks : cap);
}

// ------------------------------------------------------------------ softmax ----
// The lane-group geometry is a compile-time parameter: LPR lanes own a row (64 / LPR rows per wave), each lane
// VPL 16-byte vectors of it, LPR apart.  With constants the group reductions are DPP / lane-swap instructions
// (no general shuffles), row and vector indices need no division, and the arithmetic per element is one fma into
// exp2 for the 16-bit types.  Rows past the end are clamped to the last row on the load side and skipped on the
// store side, so the loop body has no divergent branch.  Measured against the run-time geometry it replaced:
// 46.9 vs 60 us on [1, 128, 8, 256, 256] bf16 (a plain non-temporal copy of the same bytes: 42.8 us).
constexpr int SM_WAVES = 8;       // waves per block of the vector softmax
// Stand-ins for an absent bias (zeros) or mask (ones): the kernel then reads these rows instead of branching on a
// null pointer around every load, which would keep the loads of a row group from being issued together.
// A vector row is at most 64 lanes x 8 vectors x 16 bytes.
constexpr int SM_MAXROW = 64 * 8 * 16;
__device__ __align__(16) const unsigned char sm_zero_row[SM_MAXROW] = {};
struct SmOnesRow {
    uint32_t w[SM_MAXROW / 4];
    constexpr explicit SmOnesRow(uint32_t v) : w() {
        for (int i = 0; i < SM_MAXROW / 4; ++i) w[i] = v;
    }
};
__device__ __align__(16) const SmOnesRow sm_ones_f32(0x3F800000u), sm_ones_bf16(0x3F803F80u), sm_ones_f16(0x3C003C00u);
template <typename T> __device__ __forceinline__ const T* sm_ones_row();
template <> __device__ __forceinline__ const float* sm_ones_row<float>() { return reinterpret_cast<const float*>(sm_ones_f32.w); }
template <> __device__ __forceinline__ const bf16_t* sm_ones_row<bf16_t>() { return reinterpret_cast<const bf16_t*>(sm_ones_bf16.w); }
template <> __device__ __forceinline__ const f16_t* sm_ones_row<f16_t>() { return reinterpret_cast<const f16_t*>(sm_ones_f16.w); }
// RAGGED = false: the row is exactly LPR * VPL vectors, every vector offset is an immediate (one address per lane).
template <typename T, int LPR, int VPL, bool RAGGED>
__global__ __launch_bounds__(64 * SM_WAVES) void softmax_vec_kernel(T* out, const T* x,   // out may alias x
                                                                  const T* __restrict__ mask,
                                                                  const T* __restrict__ bias, unsigned rows, int cols,
                                                                  unsigned hq) {
    constexpr int VEC = DT<T>::VEC;
    constexpr int RPW = 64 / LPR;
    constexpr bool F32 = sizeof(T) == 4;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int sub = lane / LPR;
    const int j = lane % LPR;
    const int nvec = RAGGED ? cols / VEC : LPR * VPL;
    const int rowlen = RAGGED ? cols : LPR * VPL * VEC;
    const unsigned stride = gridDim.x * SM_WAVES * RPW;
    for (unsigned base = (blockIdx.x * SM_WAVES + wave) * RPW; base < rows; base += stride) {
        const unsigned row = base + sub;
        const bool valid = row < rows;
        const unsigned rc = valid ? row : rows - 1;
        const unsigned b2 = rc / hq;                             // 32-bit: rows < 2^31 is checked by the entry point
        const T* xr = x + (long)rc * rowlen + j * VEC;
        const T* br = (bias ? bias + (long)(rc - b2 * hq) * rowlen : reinterpret_cast<const T*>(sm_zero_row)) + j * VEC;
        const T* mr = (mask ? mask + (long)b2 * rowlen : sm_ones_row<T>()) + j * VEC;
        Vec16<T> xv[VPL], bv[VPL], mv[VPL];
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            int vo = i * LPR * VEC;
            if (RAGGED) vo = j + i * LPR < nvec ? vo : (nvec - 1 - j) * VEC;   // clamped: the copy is ignored below
            xv[i] = ld16_nt(xr + vo);
            bv[i] = ld16(br + vo);
            mv[i] = ld16(mr + vo);
        }
        float v[VPL][VEC];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            const bool in = !RAGGED || j + i * LPR < nvec;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float f = DT<T>::to_f(xv[i].e[e]) + DT<T>::to_f(bv[i].e[e]);
                if (DT<T>::to_f(mv[i].e[e]) == 0.0f) f = MASK_FILL;
                if (RAGGED) f = in ? f : -INFINITY;
                v[i][e] = f;
                mx = fmaxf(mx, f);
            }
        }
        mx = group_max(mx, LPR);
        float sum = 0.0f;
        if (F32) {
#pragma unroll
            for (int i = 0; i < VPL; ++i)
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    v[i][e] = expf(v[i][e] - mx);
                    sum += v[i][e];
                }
        } else {
            const float mxl = mx * 1.4426950408889634f;
#pragma unroll
            for (int i = 0; i < VPL; ++i)
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    v[i][e] = fast_exp2(__builtin_fmaf(v[i][e], 1.4426950408889634f, -mxl));
                    sum += v[i][e];
                }
        }
        sum = group_sum(sum, LPR);
        const float inv = F32 ? 1.0f / sum : fast_rcp(sum);
        T* orow = out + (long)rc * rowlen + j * VEC;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            Vec16<T> ov;
#pragma unroll
            for (int e = 0; e < VEC; ++e) ov.e[e] = DT<T>::from_f(v[i][e] * inv);
            if (valid && (!RAGGED || j + i * LPR < nvec)) st16_nt(orow + i * LPR * VEC, ov);
        }
    }
}

// Any row length / alignment: one wave per row, three passes over the row.
template <typename T>
__global__ __launch_bounds__(BLOCK) void softmax_generic_kernel(T* out, const T* x, const T* mask,
                                                               const T* bias, long rows, int cols, long hq) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const long stride = (long)gridDim.x * WAVES_PER_BLOCK;
    for (long row = (long)blockIdx.x * WAVES_PER_BLOCK + wave; row < rows; row += stride) {
        const T* xr = x + row * cols;
        const T* mr = mask ? mask + (row / hq) * cols : nullptr;
        const T* br = bias ? bias + (row % hq) * cols : nullptr;
        auto logit = [&](int c) -> float {
            float v = DT<T>::to_f(xr[c]);
            if (br) v += DT<T>::to_f(br[c]);
            if (mr && DT<T>::to_f(mr[c]) == 0.0f) v = MASK_FILL;
            return v;
        };
        float mx = -INFINITY;
        for (int c = lane; c < cols; c += 64) mx = fmaxf(mx, logit(c));
        mx = group_max(mx, 64);
        float sum = 0.0f;
        for (int c = lane; c < cols; c += 64) sum += exp_for<T>(logit(c) - mx);
        sum = group_sum(sum, 64);
        const float inv = 1.0f / sum;
        T* orow = out + row * cols;
        // out may alias x: every element is read (above and here) by the lane that writes it
        for (int c = lane; c < cols; c += 64) orow[c] = DT<T>::from_f(exp_for<T>(logit(c) - mx) * inv);
    }
}

template <typename T>
__global__ __launch_bounds__(BLOCK) void softmax_bwd_kernel(T* dx, const T* dy, const T* y, long rows, int cols) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const long stride = (long)gridDim.x * WAVES_PER_BLOCK;
    for (long row = (long)blockIdx.x * WAVES_PER_BLOCK + wave; row < rows; row += stride) {
        const T* yr = y + row * cols;
        const T* gr = dy + row * cols;
        float dot = 0.0f;
        for (int c = lane; c < cols; c += 64) dot += DT<T>::to_f(yr[c]) * DT<T>::to_f(gr[c]);
        dot = group_sum(dot, 64);
        T* o = dx + row * cols;
        for (int c = lane; c < cols; c += 64)
            o[c] = DT<T>::from_f((DT<T>::to_f(gr[c]) - dot) * DT<T>::to_f(yr[c]));
    }
}

template <typename T>
int softmax_launch(T* out, const T* x, const T* mask, const T* bias, long rows, long cols, long hq,
                   hipStream_t st) {
    constexpr int VEC = DT<T>::VEC;
    RowGeom g;
    const bool vec_ok = cols % VEC == 0 && ffk_aligned16(out) && ffk_aligned16(x) &&
                        (!mask || ffk_aligned16(mask)) && (!bias || ffk_aligned16(bias)) &&
                        rows < (1L << 31) - (1L << 24) &&        // the vector kernel counts rows in 32 bits
                        row_geom(cols / VEC, &g);
    if (vec_ok) {
        const long rows_per_block = (long)SM_WAVES * (64 / g.lpr);
        const long need = (rows + rows_per_block - 1) / rows_per_block;
        dim3 grid((unsigned)(need < 256L * 8 ? need : 256L * 8));      // 256 CUs x 8 blocks; grid-stride beyond
#define FFK_SM_CASE(L, V)                                                                                         \
    if (g.lpr == L && g.vpl == V) {                                                                               \
        if (cols == (long)L * V * VEC)                                                                            \
            softmax_vec_kernel<T, L, V, false><<<grid, 64 * SM_WAVES, 0, st>>>(out, x, mask, bias, (unsigned)rows, (int)cols, (unsigned)hq); \
        else                                                                                                      \
            softmax_vec_kernel<T, L, V, true><<<grid, 64 * SM_WAVES, 0, st>>>(out, x, mask, bias, (unsigned)rows, (int)cols, (unsigned)hq); \
        return ffk_check_launch("ffk_softmax_fwd");                                                               \
    }
        FFK_ROW_GEOMETRIES(FFK_SM_CASE)
#undef FFK_SM_CASE
        return ffk_fail(FFK_ERR_UNSUPPORTED, "ffk_softmax_fwd: no kernel for the row geometry (%d lanes, %d vectors)", g.lpr, g.vpl);
    } else {
        dim3 grid(row_grid(rows, 64));
        softmax_generic_kernel<T><<<grid, BLOCK, 0, st>>>(out, x, mask, bias, rows, (int)cols, hq);
    }
    return ffk_check_launch("ffk_softmax_fwd");
}

// ---------------------------------------------------------------- LayerNorm ----
// Same compile-time geometry as the softmax; RU row groups are loaded before any of them is normalised, so that a
// wave has RU * VPL 16-byte loads in flight (at 33.5 MB the whole launch lasts a few microseconds and only a few
// row groups per wave exist: the ramp is what counts).  65 536 x 128 bf16: 7.0 vs 9.6 us before (copy: 6.2 us).
constexpr int LN_RU = 4;
template <typename T, int LPR, int VPL, bool RAGGED>
__global__ __launch_bounds__(BLOCK) void layernorm_vec_kernel(T* __restrict__ out, float* __restrict__ mean_o,
                                                             float* __restrict__ rstd_o, const T* __restrict__ x,
                                                             const T* __restrict__ gamma,
                                                             const T* __restrict__ beta, unsigned rows, int cols,
                                                             float eps) {
    constexpr int VEC = DT<T>::VEC;
    constexpr int RPW = 64 / LPR;
    constexpr int RU = VPL <= 2 ? LN_RU : (VPL == 4 ? 2 : 1);      // registers: RU * VPL vectors held at once
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int sub = lane / LPR;
    const int j = lane % LPR;
    const int nvec = RAGGED ? cols / VEC : LPR * VPL;
    const int rowlen = RAGGED ? cols : LPR * VPL * VEC;
    const float inv_n = 1.0f / (float)rowlen;
    // gamma / beta stay in registers for the whole grid-stride loop
    float gm[VPL][VEC], bt[VPL][VEC];
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        const int vi = j + i * LPR;
        if (vi < nvec) {
            Vec16<T> gv = ld16(gamma + vi * VEC), bv = ld16(beta + vi * VEC);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                gm[i][e] = DT<T>::to_f(gv.e[e]);
                bt[i][e] = DT<T>::to_f(bv.e[e]);
            }
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) gm[i][e] = bt[i][e] = 0.0f;
        }
    }
    const unsigned stride = gridDim.x * WAVES_PER_BLOCK * RPW * RU;
    for (unsigned base = (blockIdx.x * WAVES_PER_BLOCK + wave) * RPW * RU; base < rows; base += stride) {
        Vec16<T> xv[RU][VPL];
#pragma unroll
        for (int u = 0; u < RU; ++u) {
            unsigned row = base + u * RPW + sub;
            row = row < rows ? row : rows - 1;                 // clamped: not stored below
            const T* xr = x + (long)row * rowlen + j * VEC;
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                int vo = i * LPR * VEC;
                if (RAGGED) vo = j + i * LPR < nvec ? vo : (nvec - 1 - j) * VEC;
                xv[u][i] = ld16_nt(xr + vo);
            }
        }
#pragma unroll
        for (int u = 0; u < RU; ++u) {
            const unsigned row = base + u * RPW + sub;
            const bool valid = row < rows;
            float v[VPL][VEC];
            float s = 0.0f;
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                const bool in = !RAGGED || j + i * LPR < nvec;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    v[i][e] = in ? DT<T>::to_f(xv[u][i].e[e]) : 0.0f;
                    s += v[i][e];
                }
            }
            const float mu = group_sum(s, LPR) * inv_n;
            float q = 0.0f;
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                const bool in = !RAGGED || j + i * LPR < nvec;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    v[i][e] -= mu;
                    q += in ? v[i][e] * v[i][e] : 0.0f;
                }
            }
            const float var = group_sum(q, LPR) * inv_n;
            const float rs = rsqrtf(var + eps);
            T* orow = out + (long)row * rowlen + j * VEC;
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                Vec16<T> ov;
#pragma unroll
                for (int e = 0; e < VEC; ++e) ov.e[e] = DT<T>::from_f(v[i][e] * rs * gm[i][e] + bt[i][e]);
                if (valid && (!RAGGED || j + i * LPR < nvec)) st16_nt(orow + i * LPR * VEC, ov);
            }
            if (valid && j == 0) {
                if (mean_o) mean_o[row] = mu;
                if (rstd_o) rstd_o[row] = rs;
            }
        }
    }
}

template <typename T>
__global__ __launch_bounds__(BLOCK) void layernorm_generic_kernel(T* out, float* mean_o, float* rstd_o, const T* x,
                                                                 const T* gamma, const T* beta, long rows,
                                                                 int cols, float eps) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const float inv_n = 1.0f / (float)cols;
    const long stride = (long)gridDim.x * WAVES_PER_BLOCK;
    for (long row = (long)blockIdx.x * WAVES_PER_BLOCK + wave; row < rows; row += stride) {
        const T* xr = x + row * cols;
        float s = 0.0f;
        for (int c = lane; c < cols; c += 64) s += DT<T>::to_f(xr[c]);
        const float mu = group_sum(s, 64) * inv_n;
        float q = 0.0f;
        for (int c = lane; c < cols; c += 64) {
            const float d = DT<T>::to_f(xr[c]) - mu;
            q += d * d;
        }
        const float rs = rsqrtf(group_sum(q, 64) * inv_n + eps);
        T* orow = out + row * cols;
        for (int c = lane; c < cols; c += 64)
            orow[c] = DT<T>::from_f((DT<T>::to_f(xr[c]) - mu) * rs * DT<T>::to_f(gamma[c]) + DT<T>::to_f(beta[c]));
        if (lane == 0) {
            if (mean_o) mean_o[row] = mu;
            if (rstd_o) rstd_o[row] = rs;
        }
    }
}

// dx = rstd * (g - mean(g) - xhat * mean(g * xhat)),  g = dy * gamma ; dgamma += dy * xhat ; dbeta += dy
template <typename T>
__global__ __launch_bounds__(BLOCK) void layernorm_bwd_kernel(T* dx, float* dgamma, float* dbeta, const T* dy,
                                                             const T* x, const float* mean, const float* rstd,
                                                             const T* gamma, long rows, int cols,
                                                             long rows_per_wave) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const float inv_n = 1.0f / (float)cols;
    const long w = (long)blockIdx.x * WAVES_PER_BLOCK + wave;
    const long r0 = w * rows_per_wave;
    const long r1 = r0 + rows_per_wave < rows ? r0 + rows_per_wave : rows;
    // column-partial sums of this wave, kept per lane for columns lane, lane+64, ...
    for (int c0 = 0; c0 < cols; c0 += 64 * 8) {
        float pg[8], pb[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) pg[t] = pb[t] = 0.0f;
        for (long row = r0; row < r1; ++row) {
            const float mu = mean[row], rs = rstd[row];
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int c = c0 + lane + 64 * t;
                if (c < cols) {
                    const float g = DT<T>::to_f(dy[row * cols + c]);
                    pg[t] += g * (DT<T>::to_f(x[row * cols + c]) - mu) * rs;
                    pb[t] += g;
                }
            }
        }
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const int c = c0 + lane + 64 * t;
            if (c < cols && r0 < r1) {
                atomicAdd(dgamma + c, pg[t]);
                atomicAdd(dbeta + c, pb[t]);
            }
        }
    }
    for (long row = r0; row < r1; ++row) {
        const float mu = mean[row], rs = rstd[row];
        float s1 = 0.0f, s2 = 0.0f;
        for (int c = lane; c < cols; c += 64) {
            const float g = DT<T>::to_f(dy[row * cols + c]) * DT<T>::to_f(gamma[c]);
            const float xh = (DT<T>::to_f(x[row * cols + c]) - mu) * rs;
            s1 += g;
            s2 += g * xh;
        }
        s1 = group_sum(s1, 64) * inv_n;
        s2 = group_sum(s2, 64) * inv_n;
        for (int c = lane; c < cols; c += 64) {
            const float g = DT<T>::to_f(dy[row * cols + c]) * DT<T>::to_f(gamma[c]);
            const float xh = (DT<T>::to_f(x[row * cols + c]) - mu) * rs;
            dx[row * cols + c] = DT<T>::from_f(rs * (g - s1 - xh * s2));
        }
    }
}

// Vector form of the backward pass for rows of exactly LPR * VPL vectors (at most LN_BWD_MAXCOLS elements): one pass
// over x and dy with 16-byte loads, the row sums inside the lane group, and the column sums for dgamma / dbeta kept
// per lane over the whole grid-stride loop, then folded across the wave's row groups (xor shuffles), across the
// block's waves (LDS) and into the result with one atomic per column and block.
constexpr int LN_BWD_MAXCOLS = 1024;
template <typename T, int LPR, int VPL>
__global__ __launch_bounds__(BLOCK) void layernorm_bwd_vec_kernel(T* __restrict__ dx, float* dgamma, float* dbeta,
                                                                 const T* __restrict__ dy, const T* __restrict__ x,
                                                                 const float* __restrict__ mean,
                                                                 const float* __restrict__ rstd,
                                                                 const T* __restrict__ gamma, unsigned rows) {
    constexpr int VEC = DT<T>::VEC;
    constexpr int RPW = 64 / LPR;
    constexpr int ROWLEN = LPR * VPL * VEC;
    __shared__ float red[WAVES_PER_BLOCK][2][ROWLEN];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int sub = lane / LPR;
    const int j = lane % LPR;
    const float inv_n = 1.0f / (float)ROWLEN;
    float gm[VPL][VEC], pg[VPL][VEC], pb[VPL][VEC];
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        Vec16<T> gv = ld16(gamma + (j + i * LPR) * VEC);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            gm[i][e] = DT<T>::to_f(gv.e[e]);
            pg[i][e] = pb[i][e] = 0.0f;
        }
    }
    const unsigned stride = gridDim.x * WAVES_PER_BLOCK * RPW;
    for (unsigned base = (blockIdx.x * WAVES_PER_BLOCK + wave) * RPW; base < rows; base += stride) {
        const unsigned row = base + sub;
        const bool valid = row < rows;
        const unsigned rc = valid ? row : rows - 1;              // clamped: neither stored nor accumulated below
        const T* xr = x + (long)rc * ROWLEN + j * VEC;
        const T* gr = dy + (long)rc * ROWLEN + j * VEC;
        Vec16<T> xv[VPL], dv[VPL];
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            xv[i] = ld16_nt(xr + i * LPR * VEC);
            dv[i] = ld16_nt(gr + i * LPR * VEC);
        }
        const float mu = mean[rc], rs = rstd[rc];
        float xh[VPL][VEC], g[VPL][VEC];
        float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float d = valid ? DT<T>::to_f(dv[i].e[e]) : 0.0f;
                xh[i][e] = (DT<T>::to_f(xv[i].e[e]) - mu) * rs;
                g[i][e] = d * gm[i][e];
                s1 += g[i][e];
                s2 += g[i][e] * xh[i][e];
                pg[i][e] += d * xh[i][e];
                pb[i][e] += d;
            }
        }
        s1 = group_sum(s1, LPR) * inv_n;
        s2 = group_sum(s2, LPR) * inv_n;
        T* orow = dx + (long)rc * ROWLEN + j * VEC;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            Vec16<T> ov;
#pragma unroll
            for (int e = 0; e < VEC; ++e) ov.e[e] = DT<T>::from_f(rs * (g[i][e] - s1 - xh[i][e] * s2));
            if (valid) st16_nt(orow + i * LPR * VEC, ov);
        }
    }
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
#pragma unroll
            for (int off = LPR; off < 64; off <<= 1) {
                pg[i][e] += __shfl_xor(pg[i][e], off, 64);
                pb[i][e] += __shfl_xor(pb[i][e], off, 64);
            }
            if (sub == 0) {
                red[wave][0][(j + i * LPR) * VEC + e] = pg[i][e];
                red[wave][1][(j + i * LPR) * VEC + e] = pb[i][e];
            }
        }
    }
    __syncthreads();
    for (int c = threadIdx.x; c < ROWLEN; c += BLOCK) {
        float a = 0.0f, b = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES_PER_BLOCK; ++w) {
            a += red[w][0][c];
            b += red[w][1][c];
        }
        atomicAdd(dgamma + c, a);
        atomicAdd(dbeta + c, b);
    }
}

template <typename T>
bool layernorm_bwd_vec_launch(T* dx, float* dgamma, float* dbeta, const T* dy, const T* x, const float* mean,
                              const float* rstd, const T* gamma, long rows, long cols, hipStream_t st) {
    constexpr int VEC = DT<T>::VEC;
    RowGeom g;
    if (cols % VEC != 0 || cols > LN_BWD_MAXCOLS || !ffk_aligned16(dx) || !ffk_aligned16(dy) || !ffk_aligned16(x) ||
        !ffk_aligned16(gamma) || rows >= (1L << 31) - (1L << 24) || !row_geom(cols / VEC, &g) ||
        cols != (long)g.lpr * g.vpl * VEC)
        return false;
    const long rows_per_block = (long)WAVES_PER_BLOCK * (64 / g.lpr);
    const long need = (rows + rows_per_block - 1) / rows_per_block;
    dim3 grid((unsigned)(need < 256L * 2 ? need : 256L * 2));
#define FFK_LNB_CASE(L, V)                                                                                            \
    if (g.lpr == L && g.vpl == V && (long)L * V * VEC <= LN_BWD_MAXCOLS) {                                            \
        layernorm_bwd_vec_kernel<T, L, (L * V * VEC <= LN_BWD_MAXCOLS ? V : 1)><<<grid, BLOCK, 0, st>>>(             \
            dx, dgamma, dbeta, dy, x, mean, rstd, gamma, (unsigned)rows);                                             \
        return true;                                                                                                  \
    }
    FFK_ROW_GEOMETRIES(FFK_LNB_CASE)
#undef FFK_LNB_CASE
    return false;
}

template <typename T>
int layernorm_launch(T* out, float* mean, float* rstd, const T* x, const T* gamma, const T* beta, long rows,
                     long cols, float eps, hipStream_t st) {
    constexpr int VEC = DT<T>::VEC;
    RowGeom g;
    const bool vec_ok = cols % VEC == 0 && ffk_aligned16(out) && ffk_aligned16(x) && ffk_aligned16(gamma) &&
                        ffk_aligned16(beta) && rows < (1L << 31) - (1L << 24) && row_geom(cols / VEC, &g);
    if (vec_ok) {
        const int ru = g.vpl <= 2 ? LN_RU : (g.vpl == 4 ? 2 : 1);
        const long rows_per_block = (long)WAVES_PER_BLOCK * (64 / g.lpr) * ru;
        const long need = (rows + rows_per_block - 1) / rows_per_block;
        dim3 grid((unsigned)(need < 256L * 8 ? need : 256L * 8));
#define FFK_LN_CASE(L, V)                                                                                             \
    if (g.lpr == L && g.vpl == V) {                                                                                   \
        if (cols == (long)L * V * VEC)                                                                                \
            layernorm_vec_kernel<T, L, V, false><<<grid, BLOCK, 0, st>>>(out, mean, rstd, x, gamma, beta, (unsigned)rows, (int)cols, eps); \
        else                                                                                                          \
            layernorm_vec_kernel<T, L, V, true><<<grid, BLOCK, 0, st>>>(out, mean, rstd, x, gamma, beta, (unsigned)rows, (int)cols, eps); \
        return ffk_check_launch("ffk_layernorm_fwd");                                                                 \
    }
        FFK_ROW_GEOMETRIES(FFK_LN_CASE)
#undef FFK_LN_CASE
        return ffk_fail(FFK_ERR_UNSUPPORTED, "ffk_layernorm_fwd: no kernel for the row geometry (%d lanes, %d vectors)", g.lpr, g.vpl);
    } else {
        dim3 grid(row_grid(rows, 64));
        layernorm_generic_kernel<T><<<grid, BLOCK, 0, st>>>(out, mean, rstd, x, gamma, beta, rows, (int)cols, eps);
    }
    return ffk_check_launch("ffk_layernorm_fwd");
}

// -------------------------------------------------------------- elementwise ----
// kind 0: sigmoid(a + bias) * b          (a = y, b = z)
// kind 1: c + (a + bias) * dm            (a = x, c = residual)
// kind 2: c + dm * (b * (a + bias))      (a = ab, b = g, c = z_raw)
template <typename T, int KIND>
__global__ __launch_bounds__(BLOCK) void eltwise_kernel(T* __restrict__ out, const T* __restrict__ a,
                                                       const T* __restrict__ bias, const T* __restrict__ b,
                                                       const T* __restrict__ c, const T* __restrict__ dm,
                                                       long n_rows, int C, long I, long J, long dm_sb, long dm_si,
                                                       long dm_sj, bool vec) {
    constexpr int VEC = DT<T>::VEC;
    const int per_row = vec ? C / VEC : C;
    const long total = n_rows * per_row;
    for (long idx = (long)blockIdx.x * BLOCK + threadIdx.x; idx < total; idx += (long)gridDim.x * BLOCK) {
        const long row = idx / per_row;
        const int col = (int)(idx - row * per_row) * (vec ? VEC : 1);
        const long off = row * C + col;
        const T* dmp = nullptr;
        if (dm) {
            const long jj = row % J, ii = (row / J) % I, bb = row / (J * I);
            dmp = dm + bb * dm_sb + ii * dm_si + jj * dm_sj + col;
        }
        auto f = [&](float av, float bias_v, float bv, float cv, float dv) -> float {
            if (KIND == 0) return sigmoid_f(av + bias_v) * bv;
            if (KIND == 1) return cv + (av + bias_v) * dv;
            return cv + dv * (bv * (av + bias_v));
        };
        if (vec) {
            Vec16<T> av = ld16(a + off), biasv = ld16(bias + col), bv, cv, dv, ov;
            if (KIND != 1) bv = ld16(b + off);
            if (KIND != 0) cv = ld16(c + off);
            if (dmp) dv = ld16(dmp);
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                ov.e[e] = DT<T>::from_f(f(DT<T>::to_f(av.e[e]), DT<T>::to_f(biasv.e[e]),
                                          KIND != 1 ? DT<T>::to_f(bv.e[e]) : 0.0f,
                                          KIND != 0 ? DT<T>::to_f(cv.e[e]) : 0.0f,
                                          dmp ? DT<T>::to_f(dv.e[e]) : 1.0f));
            st16(out + off, ov);
        } else {
            out[off] = DT<T>::from_f(f(DT<T>::to_f(a[off]), DT<T>::to_f(bias[col]),
                                       KIND != 1 ? DT<T>::to_f(b[off]) : 0.0f,
                                       KIND != 0 ? DT<T>::to_f(c[off]) : 0.0f,
                                       dmp ? DT<T>::to_f(dmp[0]) : 1.0f));
        }
    }
}

template <typename T, int KIND>
int eltwise_launch(void* out, const void* a, const void* bias, const void* b, const void* c, const void* dm,
                   long B, long I, long J, long C, long dm_sb, long dm_si, long dm_sj, hipStream_t st,
                   const char* name) {
    constexpr int VEC = DT<T>::VEC;
    const long n_rows = B * I * J;
    bool vec = C % VEC == 0 && ffk_aligned16(out) && ffk_aligned16(a) && ffk_aligned16(bias) &&
               (!b || ffk_aligned16(b)) && (!c || ffk_aligned16(c));
    if (dm) vec = vec && ffk_aligned16(dm) && dm_sb % VEC == 0 && dm_si % VEC == 0 && dm_sj % VEC == 0;
    const long total = n_rows * (vec ? C / VEC : C);
    long blocks = (total + BLOCK - 1) / BLOCK;
    if (blocks > 256L * 32) blocks = 256L * 32;
    eltwise_kernel<T, KIND><<<dim3((int)blocks), BLOCK, 0, st>>>((T*)out, (const T*)a, (const T*)bias, (const T*)b,
                                                              (const T*)c, (const T*)dm, n_rows, (int)C, I, J,
                                                              dm_sb, dm_si, dm_sj, vec);
    return ffk_check_launch(name);
}

template <int KIND>
int eltwise_dispatch(int dtype, void* out, const void* a, const void* bias, const void* b, const void* c,
                     const void* dm, long B, long I, long J, long C, long dm_sb, long dm_si, long dm_sj,
                     void* stream, const char* name) {
    FFK_REQUIRE(out && a && bias, FFK_ERR_NULL, "%s: null pointer", name);
    FFK_REQUIRE(KIND == 1 || b, FFK_ERR_NULL, "%s: null pointer", name);
    FFK_REQUIRE(KIND == 0 || c, FFK_ERR_NULL, "%s: null pointer", name);
    FFK_REQUIRE(B > 0 && I > 0 && J > 0 && C > 0 && C < (1L << 30), FFK_ERR_SHAPE, "%s: bad shape [%ld,%ld,%ld,%ld]",
                name, B, I, J, C);
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case FFK_F32: return eltwise_launch<float, KIND>(out, a, bias, b, c, dm, B, I, J, C, dm_sb, dm_si, dm_sj, st, name);
        case FFK_BF16: return eltwise_launch<bf16_t, KIND>(out, a, bias, b, c, dm, B, I, J, C, dm_sb, dm_si, dm_sj, st, name);
        case FFK_F16: return eltwise_launch<f16_t, KIND>(out, a, bias, b, c, dm, B, I, J, C, dm_sb, dm_si, dm_sj, st, name);
        default: return ffk_fail(FFK_ERR_DTYPE, "%s: unsupported dtype tag %d", name, dtype);
    }
}

}  // namespace

// -------------------------------------------------------------------- C ABI ----
// Plain streaming copy with the access pattern of the row kernels (16-byte non-temporal loads and stores, four
// vectors in flight per lane): what a read-once / write-once stream of a given size reaches on this GPU.
namespace {
__global__ __launch_bounds__(BLOCK) void stream_copy_kernel(u32x4* __restrict__ dst, const u32x4* __restrict__ src, long n) {
    constexpr int U = 4;
    const long stride = (long)gridDim.x * BLOCK * U;
    for (long i = (long)blockIdx.x * BLOCK * U + threadIdx.x; i < n; i += stride) {
        u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const long k = i + u * BLOCK;
            if (k < n) v[u] = __builtin_nontemporal_load(src + k);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const long k = i + u * BLOCK;
            if (k < n) __builtin_nontemporal_store(v[u], dst + k);
        }
    }
}
}  // namespace

extern "C" int ffk_stream_copy(void* dst, const void* src, int64_t bytes, void* stream) {
    FFK_REQUIRE(dst && src, FFK_ERR_NULL, "ffk_stream_copy: null pointer");
    FFK_REQUIRE(bytes > 0 && bytes % 16 == 0, FFK_ERR_SHAPE, "ffk_stream_copy: size %ld is not a positive multiple of 16", (long)bytes);
    FFK_REQUIRE(ffk_aligned16(dst) && ffk_aligned16(src), FFK_ERR_ALIGN, "ffk_stream_copy: buffers must be 16-byte aligned");
    const long n = bytes / 16;
    long blocks = (n + BLOCK * 4 - 1) / (BLOCK * 4);
    if (blocks > 256L * 16) blocks = 256L * 16;
    stream_copy_kernel<<<dim3((unsigned)blocks), BLOCK, 0, (hipStream_t)stream>>>((u32x4*)dst, (const u32x4*)src, n);
    return ffk_check_launch("ffk_stream_copy");
}

extern "C" int ffk_softmax_fwd(void* out, const void* x, const void* mask, const void* bias, int64_t B1,
                               int64_t B2, int64_t H, int64_t Nq, int64_t Nk, int dtype, void* stream) {
    FFK_REQUIRE(out && x, FFK_ERR_NULL, "ffk_softmax_fwd: null pointer");
    FFK_REQUIRE(B1 > 0 && B2 > 0 && H > 0 && Nq > 0 && Nk > 0 && Nk < (1L << 30), FFK_ERR_SHAPE,
                "ffk_softmax_fwd: bad shape [%ld,%ld,%ld,%ld,%ld]", (long)B1, (long)B2, (long)H, (long)Nq, (long)Nk);
    const long rows = B1 * B2 * H * Nq;
    // mask row = row / (H*Nq) indexes [B1*B2]; bias row = row % (H*Nq) only when B1 == 1, else
    // bias is [B1,1,H,Nq,Nk] and the B1 index must be kept: fold it by treating each b1 separately.
    hipStream_t st = (hipStream_t)stream;
    const long hq = H * Nq;
    const size_t esz = dtype == FFK_F32 ? 4 : 2;
    for (int64_t b1 = 0; b1 < B1; ++b1) {
        const long r = B2 * hq;
        const size_t xoff = (size_t)b1 * r * Nk * esz;
        void* o = (char*)out + xoff;
        const void* xi = (const char*)x + xoff;
        const void* mi = mask ? (const char*)mask + (size_t)b1 * B2 * Nk * esz : nullptr;
        const void* bi = bias ? (const char*)bias + (size_t)b1 * hq * Nk * esz : nullptr;
        int rc;
        switch (dtype) {
            case FFK_F32: rc = softmax_launch<float>((float*)o, (const float*)xi, (const float*)mi, (const float*)bi, r, Nk, hq, st); break;
            case FFK_BF16: rc = softmax_launch<bf16_t>((bf16_t*)o, (const bf16_t*)xi, (const bf16_t*)mi, (const bf16_t*)bi, r, Nk, hq, st); break;
            case FFK_F16: rc = softmax_launch<f16_t>((f16_t*)o, (const f16_t*)xi, (const f16_t*)mi, (const f16_t*)bi, r, Nk, hq, st); break;
            default: return ffk_fail(FFK_ERR_DTYPE, "ffk_softmax_fwd: unsupported dtype tag %d", dtype);
        }
        if (rc) return rc;
    }
    (void)rows;
    return FFK_OK;
}

extern "C" int ffk_softmax_bwd(void* dx, const void* dy, const void* y, int64_t rows, int64_t cols, int dtype,
                               void* stream) {
    FFK_REQUIRE(dx && dy && y, FFK_ERR_NULL, "ffk_softmax_bwd: null pointer");
    FFK_REQUIRE(rows > 0 && cols > 0 && cols < (1L << 30), FFK_ERR_SHAPE, "ffk_softmax_bwd: bad shape [%ld,%ld]",
                (long)rows, (long)cols);
    hipStream_t st = (hipStream_t)stream;
    dim3 grid(row_grid(rows, 64));
    switch (dtype) {
        case FFK_F32: softmax_bwd_kernel<float><<<grid, BLOCK, 0, st>>>((float*)dx, (const float*)dy, (const float*)y, rows, (int)cols); break;
        case FFK_BF16: softmax_bwd_kernel<bf16_t><<<grid, BLOCK, 0, st>>>((bf16_t*)dx, (const bf16_t*)dy, (const bf16_t*)y, rows, (int)cols); break;
        case FFK_F16: softmax_bwd_kernel<f16_t><<<grid, BLOCK, 0, st>>>((f16_t*)dx, (const f16_t*)dy, (const f16_t*)y, rows, (int)cols); break;
        default: return ffk_fail(FFK_ERR_DTYPE, "ffk_softmax_bwd: unsupported dtype tag %d", dtype);
    }
    return ffk_check_launch("ffk_softmax_bwd");
}

extern "C" int ffk_layernorm_fwd(void* out, float* mean, float* rstd, const void* x, const void* gamma,
                                 const void* beta, int64_t rows, int64_t cols, float eps, int dtype, void* stream) {
    FFK_REQUIRE(out && x && gamma && beta, FFK_ERR_NULL, "ffk_layernorm_fwd: null pointer");
    FFK_REQUIRE(rows > 0 && cols > 0 && cols < (1L << 30), FFK_ERR_SHAPE, "ffk_layernorm_fwd: bad shape [%ld,%ld]",
                (long)rows, (long)cols);
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case FFK_F32: return layernorm_launch<float>((float*)out, mean, rstd, (const float*)x, (const float*)gamma, (const float*)beta, rows, cols, eps, st);
        case FFK_BF16: return layernorm_launch<bf16_t>((bf16_t*)out, mean, rstd, (const bf16_t*)x, (const bf16_t*)gamma, (const bf16_t*)beta, rows, cols, eps, st);
        case FFK_F16: return layernorm_launch<f16_t>((f16_t*)out, mean, rstd, (const f16_t*)x, (const f16_t*)gamma, (const f16_t*)beta, rows, cols, eps, st);
        default: return ffk_fail(FFK_ERR_DTYPE, "ffk_layernorm_fwd: unsupported dtype tag %d", dtype);
    }
}

extern "C" int ffk_layernorm_bwd(void* dx, float* dgamma, float* dbeta, const void* dy, const void* x,
                                 const float* mean, const float* rstd, const void* gamma, int64_t rows,
                                 int64_t cols, int dtype, void* stream) {
    FFK_REQUIRE(dx && dgamma && dbeta && dy && x && mean && rstd && gamma, FFK_ERR_NULL,
                "ffk_layernorm_bwd: null pointer");
    FFK_REQUIRE(rows > 0 && cols > 0 && cols < (1L << 30), FFK_ERR_SHAPE, "ffk_layernorm_bwd: bad shape [%ld,%ld]",
                (long)rows, (long)cols);
    hipStream_t st = (hipStream_t)stream;
    bool done = false;
    switch (dtype) {
        case FFK_F32: done = layernorm_bwd_vec_launch<float>((float*)dx, dgamma, dbeta, (const float*)dy, (const float*)x, mean, rstd, (const float*)gamma, rows, cols, st); break;
        case FFK_BF16: done = layernorm_bwd_vec_launch<bf16_t>((bf16_t*)dx, dgamma, dbeta, (const bf16_t*)dy, (const bf16_t*)x, mean, rstd, (const bf16_t*)gamma, rows, cols, st); break;
        case FFK_F16: done = layernorm_bwd_vec_launch<f16_t>((f16_t*)dx, dgamma, dbeta, (const f16_t*)dy, (const f16_t*)x, mean, rstd, (const f16_t*)gamma, rows, cols, st); break;
        default: return ffk_fail(FFK_ERR_DTYPE, "ffk_layernorm_bwd: unsupported dtype tag %d", dtype);
    }
    if (done) return ffk_check_launch("ffk_layernorm_bwd");
    const long waves = 256L * 8 * WAVES_PER_BLOCK;
    const long rpw = (rows + waves - 1) / waves;
    const long nw = (rows + rpw - 1) / rpw;
    dim3 grid((int)((nw + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK));
    switch (dtype) {
        case FFK_F32: layernorm_bwd_kernel<float><<<grid, BLOCK, 0, st>>>((float*)dx, dgamma, dbeta, (const float*)dy, (const float*)x, mean, rstd, (const float*)gamma, rows, (int)cols, rpw); break;
        case FFK_BF16: layernorm_bwd_kernel<bf16_t><<<grid, BLOCK, 0, st>>>((bf16_t*)dx, dgamma, dbeta, (const bf16_t*)dy, (const bf16_t*)x, mean, rstd, (const bf16_t*)gamma, rows, (int)cols, rpw); break;
        case FFK_F16: layernorm_bwd_kernel<f16_t><<<grid, BLOCK, 0, st>>>((f16_t*)dx, dgamma, dbeta, (const f16_t*)dy, (const f16_t*)x, mean, rstd, (const f16_t*)gamma, rows, (int)cols, rpw); break;
        default: return ffk_fail(FFK_ERR_DTYPE, "ffk_layernorm_bwd: unsupported dtype tag %d", dtype);
    }
    return ffk_check_launch("ffk_layernorm_bwd");
}

extern "C" int ffk_bias_sigmoid_mul(void* out, const void* y, const void* bias, const void* z, int64_t rows,
                                    int64_t C, int dtype, void* stream) {
    return eltwise_dispatch<0>(dtype, out, y, bias, z, nullptr, nullptr, 1, 1, rows, C, 0, 0, 0, stream,
                               "ffk_bias_sigmoid_mul");
}

extern "C" int ffk_bias_dropout_add(void* out, const void* x, const void* bias, const void* dm,
                                    const void* residual, int64_t B, int64_t I, int64_t J, int64_t C,
                                    int64_t dm_sb, int64_t dm_si, int64_t dm_sj, int dtype, void* stream) {
    return eltwise_dispatch<1>(dtype, out, x, bias, nullptr, residual, dm, B, I, J, C, dm_sb, dm_si, dm_sj, stream,
                               "ffk_bias_dropout_add");
}

extern "C" int ffk_bias_ele_dropout_res(void* out, const void* ab, const void* bias, const void* g, const void* dm,
                                        const void* z_raw, int64_t B, int64_t I, int64_t J, int64_t C,
                                        int64_t dm_sb, int64_t dm_si, int64_t dm_sj, int dtype, void* stream) {
    return eltwise_dispatch<2>(dtype, out, ab, bias, g, z_raw, dm, B, I, J, C, dm_sb, dm_si, dm_sj, stream,
                               "ffk_bias_ele_dropout_res");
}
