// Weights-stationary variant of the fused linear layer (see ffk_fused_linear in include/ffk.h),
// bf16, K = 64, 128 or 256: the projections of the pair and MSA stacks (and of the extra-MSA and
// template stacks at 64 channels), where M is 10^5 .. 10^6 rows and the whole weight matrix is a few
// hundred KB.
//
// One persistent workgroup of 8 wavefronts per CU.  The weight matrix is split into "slots" of 32
// output rows; every wave keeps the MFMA fragments of up to three slots in registers for the whole
// kernel, so weights are read from memory exactly once per workgroup.  Rows of A stream through a
// double-buffered 128-row slab in LDS: global -> registers -> (LayerNorm in registers, 16 lanes
// per row) -> LDS, the loads of slab i+1 being in flight while slab i is multiplied.  Each wave
// multiplies every 32-row group of the slab against its own slots and finishes the resulting
// 32x32 blocks straight from the accumulator registers - bias, activation, GLU, row mask, gate
// and residual - and stores them without LDS staging:
//   * tiles that are contiguous along channels (plain [row][channel] outputs, q / k / gate tiles)
//     use the product W . A^T, so a lane owns one row and 4 x 4 consecutive channels;
//   * tiles that are contiguous along rows (v tiles, channel-major outputs) use A . W^T, so a
//     lane owns one channel and 4 x 4 consecutive rows.
// Attention operand tiles are written as 32 contiguous bytes per lane, the order in which the
// attention kernel loads them.
#include "ffk_common.h"
#include <stdlib.h>
#include <type_traits>

namespace {

constexpr int WS_WAVES = 8;
constexpr int WS_THREADS = 64 * WS_WAVES;
constexpr int WS_NS = 4;                 // weight slots per wave: up to 4 (K = 64), 3 (K = 128), 2 (K = 256, 64 registers a slot)
constexpr int WS_MAX_GRID = 256;         // one workgroup per CU
// Per-K geometry: a slab is as many rows as 512 threads fetch with four 16-byte loads each.
template <int K> struct WsGeo {
    static constexpr int KS = K / 16;                // MFMA K steps
    static constexpr int AP = K * 2 + 16;            // LDS row pitch in bytes
    static constexpr int LPR = K / 8;                // lanes (16-byte vectors) per row
    static constexpr int RPP = WS_THREADS / LPR;     // rows fetched per pass
    static constexpr int BM = 4 * RPP;               // rows per slab: 128 (K = 128) or 64 (K = 256)
    static constexpr int RG = BM / 32;               // 32-row groups per slab
};

typedef bf16_t T;

struct WsPlan {
    int wrow[WS_WAVES][WS_NS];   // first weight row of the slot
    int tile[WS_WAVES][WS_NS];   // descriptor tile the slot belongs to, -1 = unused
    int chan[WS_WAVES][WS_NS];   // first output channel (within the tile) of the slot's unit
    int glu[WS_WAVES][WS_NS];    // 0 plain, 1 value half of a GLU unit (gate half in the next slot), 2 gate half
    int rg_first[WS_WAVES], rg_step[WS_WAVES];   // row groups of a slab this wave works on
    int row_perm;                // 1: rows of a group are read through tau (launch has channel-major tiles)
    int mask_tile;               // first tile with a row mask (all masked tiles share its mask), -1 = none
    int max_slots;               // largest number of slots any wave holds
    int resid_a2;                // 1: every residual is the second operand itself (same rows): taken from its LDS slab
    int bias_tile;               // index of a trailing FFK_TILE_BIAS tile (<= 4 heads, K = 128), -1 = none: it takes no
                                 // weight slot - its few dot products per row are 16 x 16 x 32 MFMAs on the slab in LDS
};

struct WsArgs {
    ffk_linear_desc d;
    WsPlan plan;
};

// What the epilogue of one slot needs, copied out of the tile descriptor once per kernel so that it
// lives in scalar registers (reading descriptor fields inside the loops costs a scalar load plus a
// full wait each time).  Channel offsets of the slot's unit are folded into the pointers.
struct WsSlot {
    T* out;
    const T* resid;
    const T* gate;
    int8_t* xtail;           // tail bytes of resid / out as an extended residual stream, or nullptr
    long s_o, s_i, s_d, gate_ld;
    unsigned inner;
    unsigned gate_rows;      // 0, or the period of the gate's row index
    int ncols_left;          // valid channels from the unit's first channel on
    int kind, act;
    float scale;
    bool masked;
    bool has_bias;
};

// sigmoid(acc + b) with the bias table entry pre-multiplied:  bs = -log2(e) * b
__device__ __forceinline__ float ws_sigmoid_pre(float acc, float bs) {
    return fast_rcp(1.0f + fast_exp2(__builtin_fmaf(acc, -1.4426950408889634f, bs)));
}

// tiles stored with channels contiguous (lane = row) vs rows contiguous (lane = channel)
__host__ __device__ __forceinline__ bool ws_by_rows(const ffk_tile& t) {
    return t.kind == FFK_TILE_QK || t.kind == FFK_TILE_ACC || (t.kind == FFK_TILE_STRIDED && t.s_d == 1);
}

__device__ __forceinline__ void unpack4(const T* p, float (&f)[4]) {
    u32x2 raw = *reinterpret_cast<const u32x2*>(p);
    const T* h = reinterpret_cast<const T*>(&raw);
#pragma unroll
    for (int e = 0; e < 4; ++e) f[e] = (float)h[e];
}

// Index permutation tau(8a + 4h + b) = 16h + 4a + b.  An MFMA accumulator register v = 4a + b of
// half-wave h holds row 8a + 4h + b of the M operand; loading M-operand row i from source row tau(i)
// therefore leaves source rows 16h .. 16h + 15 in registers 0 .. 15: sixteen consecutive channels
// (or rows) per lane, i.e. 32 contiguous bytes to store.
__device__ __forceinline__ int ws_tau(int i) { return ((i >> 2) & 1) * 16 + (i >> 3) * 4 + (i & 3); }

__device__ __forceinline__ void unpack8(const T* p, float* f) {
    u32x4 raw = *reinterpret_cast<const u32x4*>(p);
    const T* h = reinterpret_cast<const T*>(&raw);
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = (float)h[e];
}

// Two forms of each epilogue.  The "compact" one funnels every bias / activation / scale combination
// through one intermediate array; the other gives each combination its own straight-line path from the
// accumulators to the rounded outputs, which executes about 30 vector instructions fewer per 32x32 block
// (no register copies where paths join, no cleared gate accumulator for plain units) but needs more
// registers.  The kernel variants with three or four weight slots or K = 256 have no registers to spare -
// there the second form spills, and a spill costs far more than it saves - so they keep the compact form.
// ---- lane = row (n32 = its row within the group), registers = channels -----------------------
// STRIDED tiles: weight rows were loaded through tau, registers hold channels 16*half + v.
// ACC / QK tiles: natural weight order, registers hold channels 8a + 4*half + b.
// sb: this slot's 32 (GLU: 64) bias values in LDS (fp32); rmask: the row's mask value.
template <bool GLU, bool XT>
__device__ __forceinline__ void ws_store_rows_compact(const WsSlot& t, const f32x16& acc, const f32x16& accg, const float* sb,
                                              bool valid, unsigned mc, unsigned hi, unsigned lo, float rmask, int half) {
    const bool strided = t.kind == FFK_TILE_STRIDED;
    float x[16];
    {
        f32x4 bv[4], bg[4];
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int o = strided ? 16 * half + 4 * a : 4 * half + 8 * a;
            bv[a] = *reinterpret_cast<const f32x4*>(sb + o);
            if (GLU) bg[a] = *reinterpret_cast<const f32x4*>(sb + 32 + o);
        }
        if (GLU) {
#pragma unroll
            for (int v = 0; v < 16; ++v) x[v] = (acc[v] + bv[v >> 2][v & 3]) * ws_sigmoid_pre(accg[v], bg[v >> 2][v & 3]);
        } else if (t.act == FFK_ACT_SIGMOID) {
#pragma unroll
            for (int v = 0; v < 16; ++v) x[v] = ws_sigmoid_pre(acc[v], bv[v >> 2][v & 3]);
        } else if (t.has_bias) {
#pragma unroll
            for (int v = 0; v < 16; ++v) x[v] = acc[v] + bv[v >> 2][v & 3];
        } else {
#pragma unroll
            for (int v = 0; v < 16; ++v) x[v] = acc[v];
        }
    }
    if (!GLU && t.act == FFK_ACT_RELU) {
#pragma unroll
        for (int v = 0; v < 16; ++v) x[v] = relu_f(x[v]);
    }
    T y[16];
    if (t.masked || t.scale != 1.0f) {
        const float scl = t.scale * rmask;
#pragma unroll
        for (int v = 0; v < 16; ++v) y[v] = (T)(x[v] * scl);
    } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) y[v] = (T)x[v];
    }

    T* out = t.out;
    if (t.kind == FFK_TILE_ACC) {
        if (valid && t.ncols_left >= 32) {
            T* p = out + (long)hi * t.s_o + (long)(lo >> 5) * 1024 + ((half * 32 + (lo & 31)) << 4);
            *reinterpret_cast<u32x4*>(p) = *reinterpret_cast<const u32x4*>(&y[0]);
            *reinterpret_cast<u32x4*>(p + 8) = *reinterpret_cast<const u32x4*>(&y[8]);
        }
    } else if (t.kind == FFK_TILE_QK) {
        if (valid && t.ncols_left >= 32) {
            T* p = out + (long)hi * t.s_o + (long)(lo >> 5) * 1024 + (lo & 31) * 16 + 4 * half;
#pragma unroll
            for (int a = 0; a < 4; ++a)      // d = 8a + 4 half + b  ->  (d >> 4) * 512 + n * 16 + (d & 15)
                *reinterpret_cast<u32x2*>(p + (a >> 1) * 512 + (a & 1) * 8) = *reinterpret_cast<const u32x2*>(&y[4 * a]);
        }
    } else {
        const int cl = 16 * half;                        // this lane's 16 channels, relative to the unit
        const long off = (long)hi * t.s_o + (long)lo * t.s_i + cl;
        const bool ok0 = valid && cl + 8 <= t.ncols_left, ok1 = valid && cl + 16 <= t.ncols_left;
        if (t.gate || t.resid) {
            // every load first (clamped, unconditional), then combine and store
            u32x4 gv[2], rv[2];
            const T* gate = t.gate ? t.gate + (long)(t.gate_rows ? mc % t.gate_rows : mc) * t.gate_ld + cl : nullptr;
            const T* resid = t.resid ? t.resid + off : nullptr;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int cj = cl + 8 * j + 8 <= t.ncols_left ? 8 * j : (cl + 8 <= t.ncols_left ? 0 : -cl);
                if (gate) gv[j] = *reinterpret_cast<const u32x4*>(gate + cj);
                if (resid) rv[j] = *reinterpret_cast<const u32x4*>(resid + cj);
            }
            if (XT && t.xtail) {     // extended residual stream (whole 16-channel runs: ncols % 16 == 0 with a tail)
                const u32x4 tv = *reinterpret_cast<const u32x4*>(t.xtail + (ok1 ? off : off - cl));
                u32x4 tn;
#pragma unroll
                for (int j = 0; j < 2; ++j) {       // eight channels at a time (register budget)
                    float f[8];
                    xs_decode8(rv[j], tv[2 * j], tv[2 * j + 1], f);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        float u = (float)y[8 * j + e];
                        if (gate) u = (float)(T)(u * (float)reinterpret_cast<const T*>(&gv[j])[e]);
                        f[e] += u;
                    }
                    u32x4 hv;
                    uint32_t ta, tb;
                    xs_encode8(f, hv, ta, tb);
                    tn[2 * j] = ta;
                    tn[2 * j + 1] = tb;
                    if (ok1) *reinterpret_cast<u32x4*>(out + off + 8 * j) = hv;
                }
                if (ok1) *reinterpret_cast<u32x4*>(t.xtail + off) = tn;
                return;
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const T* gh = reinterpret_cast<const T*>(&gv[j]);
                const T* rh = reinterpret_cast<const T*>(&rv[j]);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float f = (float)y[8 * j + e];
                    if (gate) f = (float)(T)(f * (float)gh[e]);
                    if (resid) f += (float)rh[e];
                    y[8 * j + e] = (T)f;
                }
            }
        }
        if (ok0) *reinterpret_cast<u32x4*>(out + off) = *reinterpret_cast<const u32x4*>(&y[0]);
        if (ok1) *reinterpret_cast<u32x4*>(out + off + 8) = *reinterpret_cast<const u32x4*>(&y[8]);
    }
}

// ---- lane = channel, registers = rows ----------------------------------------------------------
// V tiles: natural row order (registers hold rows 8a + 4*half + b of the group).
// STRIDED (channel-major) tiles: the A fragments were loaded through tau, registers hold rows
// 16*half + v: sixteen consecutive rows, which never straddle `inner` (inner % 16 == 0, M % 16 == 0).
// sm: mask values (fp32, LDS) of the group's 32 rows, or nullptr.
template <bool GLU>
__device__ __forceinline__ void ws_store_cols_compact(const WsSlot& t, const f32x16& acc, const f32x16& accg, const float* sb,
                                              const float* sm, long m0g, int M, int l32, int half) {
    const float bv = sb[l32], bg = GLU ? sb[32 + l32] : 0.0f;
    float x[16];
    if (GLU) {
#pragma unroll
        for (int v = 0; v < 16; ++v) x[v] = (acc[v] + bv) * ws_sigmoid_pre(accg[v], bg);
    } else if (t.act == FFK_ACT_SIGMOID) {
#pragma unroll
        for (int v = 0; v < 16; ++v) x[v] = ws_sigmoid_pre(acc[v], bv);
    } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) x[v] = acc[v] + bv;
        if (t.act == FFK_ACT_RELU) {
#pragma unroll
            for (int v = 0; v < 16; ++v) x[v] = relu_f(x[v]);
        }
    }

    T* out = t.out;
    const bool vt = t.kind == FFK_TILE_V;
    const long mr = vt ? m0g : m0g + 16 * half;          // V: the group is one whole key tile (inner % 32 == 0)
    const bool ok = mr < M;
    const unsigned mc = (unsigned)(ok ? mr : 0);
    unsigned hi = 0, lo = mc;
    if (t.inner < (unsigned)M) {
        hi = mc / t.inner;
        lo = mc - hi * t.inner;
    }
    // the mask multiply is skipped for row groups without a masked row (the common case)
    if (sm && !vt && __builtin_amdgcn_ballot_w64(sm[l32] != 1.0f) != 0) {
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const f32x4 mk = *reinterpret_cast<const f32x4*>(sm + 16 * half + 4 * a);
#pragma unroll
            for (int b = 0; b < 4; ++b) x[4 * a + b] *= mk[b];
        }
    }
    T y[16];
    if (t.scale != 1.0f) {
#pragma unroll
        for (int v = 0; v < 16; ++v) y[v] = (T)(x[v] * t.scale);
    } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) y[v] = (T)x[v];
    }
    if (vt) {
        if (ok && t.ncols_left >= 32) {
            T* p = out + (long)hi * t.s_o + (long)(lo >> 5) * 1024 + ((half * 32 + l32) << 4);
            *reinterpret_cast<u32x4*>(p) = *reinterpret_cast<const u32x4*>(&y[0]);
            *reinterpret_cast<u32x4*>(p + 8) = *reinterpret_cast<const u32x4*>(&y[8]);
        }
    } else if (ok && l32 < t.ncols_left) {
        T* p = out + (long)hi * t.s_o + lo + (long)l32 * t.s_d;
        *reinterpret_cast<u32x4*>(p) = *reinterpret_cast<const u32x4*>(&y[0]);
        *reinterpret_cast<u32x4*>(p + 8) = *reinterpret_cast<const u32x4*>(&y[8]);
    }
}

// ---- lane = row (n32 = its row within the group), registers = channels -----------------------
// STRIDED tiles: weight rows were loaded through tau, registers hold channels 16*half + v.
// ACC / QK tiles: natural weight order, registers hold channels 8a + 4*half + b.
// sb: this slot's 32 (GLU: 64) bias values in LDS (fp32); rmask: the row's mask value.
template <bool GLU, bool XT>
__device__ __forceinline__ void ws_store_rows(const WsSlot& t, const f32x16& acc, const f32x16& accg, const float* sb,
                                              bool valid, unsigned mc, unsigned hi, unsigned lo, float rmask, int half) {
    const bool strided = t.kind == FFK_TILE_STRIDED;
    // Every combination of bias / activation / scale is its own straight-line path from the accumulators
    // to the rounded outputs: a shared intermediate array makes the compiler copy the 16 registers where
    // the paths join, and the vector instruction count is what this kernel's time follows.
    T y[16];
    const bool scaled = t.masked || t.scale != 1.0f;
    const float scl = t.scale * rmask;
    auto emit = [&](auto value) {
        if (scaled) {
#pragma unroll
            for (int v = 0; v < 16; ++v) y[v] = (T)(value(v) * scl);
        } else {
#pragma unroll
            for (int v = 0; v < 16; ++v) y[v] = (T)value(v);
        }
    };
    if (GLU || t.has_bias || t.act == FFK_ACT_SIGMOID) {
        f32x4 bv[4], bg[4];
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int o = strided ? 16 * half + 4 * a : 4 * half + 8 * a;
            bv[a] = *reinterpret_cast<const f32x4*>(sb + o);
            if (GLU) bg[a] = *reinterpret_cast<const f32x4*>(sb + 32 + o);
        }
        if (GLU) {
            emit([&](int v) { return (acc[v] + bv[v >> 2][v & 3]) * ws_sigmoid_pre(accg[v], bg[v >> 2][v & 3]); });
        } else if (t.act == FFK_ACT_SIGMOID) {
            emit([&](int v) { return ws_sigmoid_pre(acc[v], bv[v >> 2][v & 3]); });
        } else if (t.act == FFK_ACT_RELU) {
            emit([&](int v) { return relu_f(acc[v] + bv[v >> 2][v & 3]); });
        } else {
            emit([&](int v) { return acc[v] + bv[v >> 2][v & 3]; });
        }
    } else if (t.act == FFK_ACT_RELU) {
        emit([&](int v) { return relu_f(acc[v]); });
    } else {
        emit([&](int v) { return acc[v]; });
    }

    T* out = t.out;
    if (t.kind == FFK_TILE_ACC) {
        if (valid && t.ncols_left >= 32) {
            T* p = out + (long)hi * t.s_o + (long)(lo >> 5) * 1024 + ((half * 32 + (lo & 31)) << 4);
            *reinterpret_cast<u32x4*>(p) = *reinterpret_cast<const u32x4*>(&y[0]);
            *reinterpret_cast<u32x4*>(p + 8) = *reinterpret_cast<const u32x4*>(&y[8]);
        }
    } else if (t.kind == FFK_TILE_QK) {
        if (valid && t.ncols_left >= 32) {
            T* p = out + (long)hi * t.s_o + (long)(lo >> 5) * 1024 + (lo & 31) * 16 + 4 * half;
#pragma unroll
            for (int a = 0; a < 4; ++a)      // d = 8a + 4 half + b  ->  (d >> 4) * 512 + n * 16 + (d & 15)
                *reinterpret_cast<u32x2*>(p + (a >> 1) * 512 + (a & 1) * 8) = *reinterpret_cast<const u32x2*>(&y[4 * a]);
        }
    } else {
        const int cl = 16 * half;                        // this lane's 16 channels, relative to the unit
        const long off = (long)hi * t.s_o + (long)lo * t.s_i + cl;
        const bool ok0 = valid && cl + 8 <= t.ncols_left, ok1 = valid && cl + 16 <= t.ncols_left;
        if (t.gate || t.resid) {
            // every load first (clamped, unconditional), then combine and store
            u32x4 gv[2], rv[2];
            const T* gate = t.gate ? t.gate + (long)(t.gate_rows ? mc % t.gate_rows : mc) * t.gate_ld + cl : nullptr;
            const T* resid = t.resid ? t.resid + off : nullptr;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int cj = cl + 8 * j + 8 <= t.ncols_left ? 8 * j : (cl + 8 <= t.ncols_left ? 0 : -cl);
                if (gate) gv[j] = *reinterpret_cast<const u32x4*>(gate + cj);
                if (resid) rv[j] = *reinterpret_cast<const u32x4*>(resid + cj);
            }
            if (XT && t.xtail) {     // extended residual stream (whole 16-channel runs: ncols % 16 == 0 with a tail)
                const u32x4 tv = *reinterpret_cast<const u32x4*>(t.xtail + (ok1 ? off : off - cl));
                u32x4 tn;
#pragma unroll
                for (int j = 0; j < 2; ++j) {       // eight channels at a time (register budget)
                    float f[8];
                    xs_decode8(rv[j], tv[2 * j], tv[2 * j + 1], f);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        float u = (float)y[8 * j + e];
                        if (gate) u = (float)(T)(u * (float)reinterpret_cast<const T*>(&gv[j])[e]);
                        f[e] += u;
                    }
                    u32x4 hv;
                    uint32_t ta, tb;
                    xs_encode8(f, hv, ta, tb);
                    tn[2 * j] = ta;
                    tn[2 * j + 1] = tb;
                    if (ok1) *reinterpret_cast<u32x4*>(out + off + 8 * j) = hv;
                }
                if (ok1) *reinterpret_cast<u32x4*>(t.xtail + off) = tn;
                return;
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const T* gh = reinterpret_cast<const T*>(&gv[j]);
                const T* rh = reinterpret_cast<const T*>(&rv[j]);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float f = (float)y[8 * j + e];
                    if (gate) f = (float)(T)(f * (float)gh[e]);
                    if (resid) f += (float)rh[e];
                    y[8 * j + e] = (T)f;
                }
            }
        }
        if (ok0) *reinterpret_cast<u32x4*>(out + off) = *reinterpret_cast<const u32x4*>(&y[0]);
        if (ok1) *reinterpret_cast<u32x4*>(out + off + 8) = *reinterpret_cast<const u32x4*>(&y[8]);
    }
}

// ---- lane = channel, registers = rows ----------------------------------------------------------
// V tiles: natural row order (registers hold rows 8a + 4*half + b of the group).
// STRIDED (channel-major) tiles: the A fragments were loaded through tau, registers hold rows
// 16*half + v: sixteen consecutive rows, which never straddle `inner` (inner % 16 == 0, M % 16 == 0).
// sm: mask values (fp32, LDS) of the group's 32 rows, or nullptr.
template <bool GLU>
__device__ __forceinline__ void ws_store_cols(const WsSlot& t, const f32x16& acc, const f32x16& accg, const float* sb,
                                              const float* sm, long m0g, int M, int l32, int half) {
    const float bv = sb[l32], bg = GLU ? sb[32 + l32] : 0.0f;
    float x[16];
    if (GLU) {
#pragma unroll
        for (int v = 0; v < 16; ++v) x[v] = (acc[v] + bv) * ws_sigmoid_pre(accg[v], bg);
    } else if (t.act == FFK_ACT_SIGMOID) {
#pragma unroll
        for (int v = 0; v < 16; ++v) x[v] = ws_sigmoid_pre(acc[v], bv);
    } else if (t.act == FFK_ACT_RELU) {
#pragma unroll
        for (int v = 0; v < 16; ++v) x[v] = relu_f(acc[v] + bv);
    } else if (t.has_bias) {
#pragma unroll
        for (int v = 0; v < 16; ++v) x[v] = acc[v] + bv;
    } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) x[v] = acc[v];
    }

    T* out = t.out;
    const bool vt = t.kind == FFK_TILE_V;
    const long mr = vt ? m0g : m0g + 16 * half;          // V: the group is one whole key tile (inner % 32 == 0)
    const bool ok = mr < M;
    const unsigned mc = (unsigned)(ok ? mr : 0);
    unsigned hi = 0, lo = mc;
    if (t.inner < (unsigned)M) {
        hi = mc / t.inner;
        lo = mc - hi * t.inner;
    }
    // the mask multiply is skipped for row groups without a masked row (the common case)
    if (sm && !vt && __builtin_amdgcn_ballot_w64(sm[l32] != 1.0f) != 0) {
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const f32x4 mk = *reinterpret_cast<const f32x4*>(sm + 16 * half + 4 * a);
#pragma unroll
            for (int b = 0; b < 4; ++b) x[4 * a + b] *= mk[b];
        }
    }
    T y[16];
    if (t.scale != 1.0f) {
#pragma unroll
        for (int v = 0; v < 16; ++v) y[v] = (T)(x[v] * t.scale);
    } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) y[v] = (T)x[v];
    }
    if (vt) {
        if (ok && t.ncols_left >= 32) {
            T* p = out + (long)hi * t.s_o + (long)(lo >> 5) * 1024 + ((half * 32 + l32) << 4);
            *reinterpret_cast<u32x4*>(p) = *reinterpret_cast<const u32x4*>(&y[0]);
            *reinterpret_cast<u32x4*>(p + 8) = *reinterpret_cast<const u32x4*>(&y[8]);
        }
    } else if (ok && l32 < t.ncols_left) {
        T* p = out + (long)hi * t.s_o + lo + (long)l32 * t.s_d;
        *reinterpret_cast<u32x4*>(p) = *reinterpret_cast<const u32x4*>(&y[0]);
        *reinterpret_cast<u32x4*>(p + 8) = *reinterpret_cast<const u32x4*>(&y[8]);
    }
}

// GLU unit of a [row][channel] tile of a second-operand launch, where both LayerNorms are folded into the
// weights (see a2 in include/ffk.h): with W' = W * gamma the normalised product is
//     W LN(x) + b = rstd * (W' x - mean * c1) + c2,   c1[n] = sum_k W'[n][k],  c2[n] = sum_k W[n][k] beta[k] + b[n],
// so the slab needs no normalisation pass at all: mean and rstd of the lane's row come from the fragments the
// products use, c2 sits in the bias table, c1 in a table of its own; the gate half does the same with the
// second operand's row.  out = resid + value * sigmoid(gate), rounded once.  sb / sc1: this unit's 64 bias
// values / 64 row sums in LDS (fp32), value half first.
template <bool XT>
__device__ __forceinline__ void ws_store_rows_folded(const WsSlot& t, const f32x16& acc, const f32x16& accg, const float* sb,
                                                     const float* sc1, float rstd, float nmr, float rstd_g, float nmr_g,
                                                     bool valid, unsigned hi, unsigned lo, int half,
                                                     const unsigned char* a2row, int a2vec, int a2swz) {
    // rstd_g / nmr_g (the second operand's statistics) arrive multiplied by -log2(e), as the gate's bias table is
    // a2row: this lane's row of the second operand's LDS slab when that operand is also the residual (the triangle
    // multiplication's output stage: gate input and residual are both z), else nullptr; a2vec: the 16-byte vector
    // of the row this lane's 16 channels start at; a2swz: the row's swizzle (vector v lives at v ^ a2swz)
    const int cl = 16 * half;
    const long off = (long)hi * t.s_o + (long)lo * t.s_i + cl;
    u32x4 rv[2];
    if (t.resid) {
        if (a2row) {
            rv[0] = *reinterpret_cast<const u32x4*>(a2row + ((a2vec ^ a2swz) << 4));
            rv[1] = *reinterpret_cast<const u32x4*>(a2row + (((a2vec + 1) ^ a2swz) << 4));
        } else {
            rv[0] = *reinterpret_cast<const u32x4*>(t.resid + off);
            rv[1] = *reinterpret_cast<const u32x4*>(t.resid + off + 8);
        }
    }
    if (XT && t.xtail) {       // extended residual stream: the update is added at 24 bits, eight channels at a time
        const u32x4 tv = *reinterpret_cast<const u32x4*>(t.xtail + off);
        u32x4 tn;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            f32x4 bv[2], bg[2], cv[2], cg[2];      // the tables of these eight channels only (register budget)
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                const int o = cl + 8 * j + 4 * a;
                bv[a] = *reinterpret_cast<const f32x4*>(sb + o);
                bg[a] = *reinterpret_cast<const f32x4*>(sb + 32 + o);
                cv[a] = *reinterpret_cast<const f32x4*>(sc1 + o);
                cg[a] = *reinterpret_cast<const f32x4*>(sc1 + 32 + o);
            }
            float f[8];
            xs_decode8(rv[j], tv[2 * j], tv[2 * j + 1], f);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int v = 8 * j + e;
                const float val = __builtin_fmaf(acc[v], rstd, __builtin_fmaf(cv[e >> 2][e & 3], nmr, bv[e >> 2][e & 3]));
                const float garg = __builtin_fmaf(accg[v], rstd_g, __builtin_fmaf(cg[e >> 2][e & 3], nmr_g, bg[e >> 2][e & 3]));
                f[e] += (float)(T)(val * fast_rcp(1.0f + fast_exp2(garg)));
            }
            u32x4 hv;
            uint32_t ta, tb;
            xs_encode8(f, hv, ta, tb);
            tn[2 * j] = ta;
            tn[2 * j + 1] = tb;
            if (valid) *reinterpret_cast<u32x4*>(t.out + off + 8 * j) = hv;
        }
        if (valid) *reinterpret_cast<u32x4*>(t.xtail + off) = tn;
        return;
    }
    f32x4 bv[4], bg[4], cv[4], cg[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        const int o = 16 * half + 4 * a;
        bv[a] = *reinterpret_cast<const f32x4*>(sb + o);
        bg[a] = *reinterpret_cast<const f32x4*>(sb + 32 + o);
        cv[a] = *reinterpret_cast<const f32x4*>(sc1 + o);
        cg[a] = *reinterpret_cast<const f32x4*>(sc1 + 32 + o);
    }
    T y[16];
    const T* rh = reinterpret_cast<const T*>(&rv[0]);
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const float val = __builtin_fmaf(acc[v], rstd, __builtin_fmaf(cv[v >> 2][v & 3], nmr, bv[v >> 2][v & 3]));
        const float garg = __builtin_fmaf(accg[v], rstd_g, __builtin_fmaf(cg[v >> 2][v & 3], nmr_g, bg[v >> 2][v & 3]));
        float x = val * fast_rcp(1.0f + fast_exp2(garg));
        if (t.resid) x += (float)rh[v];
        y[v] = (T)x;
    }
    if (valid) {
        *reinterpret_cast<u32x4*>(t.out + off) = *reinterpret_cast<const u32x4*>(&y[0]);
        *reinterpret_cast<u32x4*>(t.out + off + 8) = *reinterpret_cast<const u32x4*>(&y[8]);
    }
}

// DUAL: the gate halves of the GLU units multiply a second operand (row-major rows, own LayerNorm).  Its
// slab goes from global memory straight into LDS (unpadded 256-byte rows, 16-byte columns XOR-swizzled
// with the row index) one slab ahead and is normalised in place by the threads that requested it.
// XT: the launch has tiles with a residual tail (extended residual stream); only those instantiations carry its code
template <int NS, int WS_K, bool CM, bool DUAL, bool XT>
__global__ __launch_bounds__(WS_THREADS, 2) void linear_ws_kernel(const WsArgs args) {
    typedef Mma<T> MM;
    typedef WsGeo<WS_K> G;
    constexpr int WS_KS = G::KS, WS_AP = G::AP, WS_BM = G::BM, WS_RG = G::RG, LPR = G::LPR, RPP = G::RPP;
    constexpr bool ALLOW_GLU = NS >= 2 && WS_K <= 128;
    constexpr bool LEAN = NS == 2 && WS_K <= 128 && !DUAL;   // straight-line epilogues where the registers allow them
    constexpr int AFC = WS_K == 128 ? 8 : 4;               // A fragments held at a time (register budget)
    const ffk_linear_desc& d = args.d;
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char* s_a = smem;                                                 // [2][WS_BM][WS_AP]
    float* s_mask = reinterpret_cast<float*>(smem + 2 * WS_BM * WS_AP);        // [2][WS_BM]
    float* s_bias = s_mask + 2 * WS_BM;                                        // [n_tiles][128]
    unsigned char* s_a2 = reinterpret_cast<unsigned char*>(s_bias + FFK_MAX_TILES * 128);   // DUAL: [2][WS_BM][256 B]
    static_assert(!DUAL || (WS_K == 128 && WS_BM == 128), "the second operand is built for K = 128");
    // LayerNorm parameters that are only needed when a slab is committed wait in LDS, not in registers
    float* s_cmln = reinterpret_cast<float*>(s_a2 + (DUAL ? 2 * WS_BM * 256 : 0));          // CM: gamma[128], beta[128] (fp32)
    T* s_ln2 = reinterpret_cast<T*>(s_cmln + (CM ? 256 : 0));                               // DUAL: gamma2[128], beta2[128]
    T* s_ln1 = s_ln2 + (DUAL ? 256 : 0);                                                    // !CM: gamma[K], beta[K]
    float* s_c1 = reinterpret_cast<float*>(s_ln1 + (CM ? 0 : 2 * WS_K));                    // DUAL: folded LayerNorm row sums
    constexpr bool PB = !CM && !DUAL && !XT && WS_K == 128;    // variants that take a trailing pair-bias tile
    T* s_wb = reinterpret_cast<T*>(s_c1);                                                   // PB: [4][WS_K] head weights
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, half = lane >> 5;
    const int M = d.M;
    const T* A = (const T*)d.a;
    const T* W = (const T*)d.w;

    // ---- this wave's weight slots, resident in registers ----
    int s_tile[NS], s_chan[NS], s_glu[NS], s_wrow[NS];
    WsSlot sp[NS];
    bool by_rows[NS];
    int s_wl[NS];
    bf16x8 wf[NS][WS_KS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        s_tile[s] = args.plan.tile[wave][s];
        s_chan[s] = args.plan.chan[wave][s];
        s_glu[s] = args.plan.glu[wave][s];
        s_wrow[s] = s_tile[s] >= 0 ? args.plan.wrow[wave][s] : 0;
        // [row][channel] tiles take their weight rows through tau (16 consecutive channels per lane)
        const ffk_tile& ts = d.tiles[s_tile[s] >= 0 ? s_tile[s] : 0];
        const int wl = ts.kind == FFK_TILE_STRIDED && ts.s_d == 1 ? ws_tau(l32) : l32;
        {
            const long coff = (long)(s_chan[s] >> 5) * ts.s_h;
            sp[s].out = (T*)ts.out + coff;
            sp[s].resid = ts.resid ? (const T*)ts.resid + coff : nullptr;
            sp[s].gate = ts.gate ? (const T*)ts.gate + s_chan[s] : nullptr;
            sp[s].xtail = XT && ts.xtail ? (int8_t*)ts.xtail + coff : nullptr;
            sp[s].s_o = ts.s_o;
            sp[s].s_i = ts.s_i;
            sp[s].s_d = ts.s_d;
            sp[s].gate_ld = ts.gate_ld;
            sp[s].gate_rows = (unsigned)ts.gate_rows;
            sp[s].inner = (unsigned)ts.inner;
            sp[s].ncols_left = ts.ncols - s_chan[s];
            sp[s].kind = ts.kind;
            sp[s].act = ts.act;
            sp[s].scale = ts.scale;
            sp[s].masked = ts.rowmask != nullptr;
            sp[s].has_bias = ts.bias != nullptr;
            by_rows[s] = ws_by_rows(ts);
        }
        s_wl[s] = wl;
    }
    const int rg_first = args.plan.rg_first[wave], rg_step = args.plan.rg_step[wave];
    // launches with channel-major tiles read the rows of a group through tau (16 consecutive rows per lane)
    const int n32 = args.plan.row_perm ? ws_tau(l32) : l32;

    // ---- slab streaming: thread -> (row tid / LPR + RPP * i, 8 channels starting at 8 * (tid % LPR)) ----
    const int c8 = tid % LPR, r0 = tid / LPR;
    // DUAL launches carry both LayerNorms folded into the weights: ln_gamma is the fp32 table of row sums and
    // both slabs are used as they arrive (see ws_store_rows_folded)
    const bool folded = DUAL;
    const bool ln = d.ln_gamma != nullptr && !folded;
    // row mask of the launch (all masked tiles share it): fetched with the slab, kept in LDS as fp32
    const int mt = args.plan.mask_tile;
    const T* rm = mt >= 0 ? (const T*)d.tiles[mt].rowmask : nullptr;
    const unsigned m_inner = mt >= 0 ? (unsigned)d.tiles[mt].inner : 1u;
    const long m_so = mt >= 0 ? d.tiles[mt].m_so : 0, m_si = mt >= 0 ? d.tiles[mt].m_si : 0;
    // plain row-major operands (inner >= M) need no division per fetched vector
    const bool a_flat = d.a_inner >= M, a2_flat = DUAL && d.a2_inner >= M, m_flat = m_inner >= (unsigned)M;
    Vec16<T> pre[4];
    T pm[4];
    // Channel-major A (element (m, k) at a + k * a_cs + rowoffset(m), K = 128 or 64): a thread fetches eight
    // consecutive rows of channel k = lane % 32 + 32 cb (cb < K / 32); the two half-waves of wave w own the row
    // groups 2w and 2w + 1 of each 128-row pass of the slab (one pass at K = 128, two at K = 64), so the LayerNorm
    // reduction over k stays inside 32 lanes.  The slab is transposed on its way into LDS (2-byte stores,
    // consecutive lanes -> consecutive k of one row).
    constexpr int CMI = CM ? WS_K / 32 : 4;              // channel blocks per thread
    static_assert(!CM || WS_K == 128 || WS_K == 64, "channel-major operands are built for K = 128 and 64");
    const int cm_k = lane & 31, cm_mg = 2 * wave + (lane >> 5);
    // second operand: vector v = i * 512 + tid of a slab is row v / 16, LDS column v % 16, which holds
    // global column (v % 16) ^ (row % 16); the 16 lanes of a row are adjacent, as the LayerNorm wants them
    const int a2_col = (tid & 15) ^ ((tid >> 4) & 15);
    const unsigned lds_a2 = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)s_a2;
    auto fetch = [&](int slab, int tobuf) {
        if (DUAL) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                long m = (long)slab * WS_BM + i * 32 + (tid >> 4);
                m = m < M ? m : M - 1;
                const unsigned hi = a2_flat ? 0u : (unsigned)m / (unsigned)d.a2_inner, lo = (unsigned)m - hi * (unsigned)d.a2_inner;
                const T* gp = (const T*)d.a2 + (long)hi * d.a2_so + (long)lo * d.a2_si + a2_col * 8;
                const unsigned dst = lds_a2 + tobuf * (WS_BM * 256) + (i * WS_THREADS + wave * 64) * 16;
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gp), "s"(dst) : "memory", "m0");
#pragma clang diagnostic pop
            }
        }
        if (CM) {
#pragma unroll
            for (int rp = 0; rp < 4 / CMI; ++rp) {
                long m = (long)slab * WS_BM + (cm_mg + 16 * rp) * 8;
                m = m < M ? m : M - 8;                   // M % 8 == 0; clamped groups are never stored
                const unsigned hi = a_flat ? 0u : (unsigned)m / (unsigned)d.a_inner, lo = (unsigned)m - hi * (unsigned)d.a_inner;
                const T* base = A + (long)hi * d.a_so + lo;  // a_si == 1
#pragma unroll
                for (int cb = 0; cb < CMI; ++cb) pre[rp * CMI + cb] = ld16(base + (long)(cm_k + 32 * cb) * d.a_cs);
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            long m = (long)slab * WS_BM + r0 + RPP * i;
            m = m < M ? m : M - 1;                       // clamped: rows past the end are never stored
            const unsigned hi = a_flat ? 0u : (unsigned)m / (unsigned)d.a_inner, lo = (unsigned)m - hi * (unsigned)d.a_inner;
            pre[i] = ld16(A + (long)hi * d.a_so + (long)lo * d.a_si + c8 * 8);
            if (rm) {
                const unsigned mh = m_flat ? 0u : (unsigned)m / m_inner, ml = (unsigned)m - mh * m_inner;
                pm[i] = rm[(long)mh * m_so + (long)ml * m_si];
            }
        }
    };
    auto commit = [&](int buf) {
        unsigned char* sa = s_a + buf * (WS_BM * WS_AP);
        if (DUAL) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this thread's vectors of the second operand have landed
        if (CM) {
            if (!ln) {       // nothing to normalise here: the transposition is a plain copy
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        *reinterpret_cast<T*>(sa + ((cm_mg + 16 * (i / CMI)) * 8 + j) * WS_AP + (cm_k + 32 * (i % CMI)) * 2) = pre[i].e[j];
                return;
            }
            float f[4][8];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 8; ++j) f[i][j] = (float)pre[i].e[j];
            if (ln) {
                float cm_g[CMI], cm_b[CMI];              // gamma / beta of this lane's channels
#pragma unroll
                for (int cb = 0; cb < CMI; ++cb) {
                    cm_g[cb] = s_cmln[(lane & 31) + 32 * cb];
                    cm_b[cb] = s_cmln[WS_K + (lane & 31) + 32 * cb];
                }
#pragma unroll
                for (int rp = 0; rp < 4 / CMI; ++rp)
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        float su = 0.0f;
                        if (CMI == 4) {
                            su = (f[0][j] + f[1][j]) + (f[2][j] + f[3][j]);
                        } else {
#pragma unroll
                            for (int cb = 0; cb < CMI; ++cb) su += f[rp * CMI + cb][j];
                        }
                        const float mu = group_sum(su, 32) * (1.0f / WS_K);
                        float q = 0.0f;
#pragma unroll
                        for (int cb = 0; cb < CMI; ++cb) {
                            f[rp * CMI + cb][j] -= mu;
                            q += f[rp * CMI + cb][j] * f[rp * CMI + cb][j];
                        }
                        const float rs = rsqrtf(group_sum(q, 32) * (1.0f / WS_K) + d.ln_eps);
#pragma unroll
                        for (int cb = 0; cb < CMI; ++cb)
                            f[rp * CMI + cb][j] = f[rp * CMI + cb][j] * rs * cm_g[cb] + cm_b[cb];
                    }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    *reinterpret_cast<T*>(sa + ((cm_mg + 16 * (i / CMI)) * 8 + j) * WS_AP + (cm_k + 32 * (i % CMI)) * 2) = (T)f[i][j];
            return;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            Vec16<T> x = pre[i];
            if (ln) {
                const Vec16<T> gam = *reinterpret_cast<const Vec16<T>*>(s_ln1 + c8 * 8);
                const Vec16<T> bet = *reinterpret_cast<const Vec16<T>*>(s_ln1 + WS_K + c8 * 8);
                float f[8], s = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    f[e] = (float)x.e[e];
                    s += f[e];
                }
                const float mu = group_sum(s, LPR) * (1.0f / WS_K);
                float q = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    f[e] -= mu;
                    q += f[e] * f[e];
                }
                const float rs = rsqrtf(group_sum(q, LPR) * (1.0f / WS_K) + d.ln_eps);
#pragma unroll
                for (int e = 0; e < 8; ++e) x.e[e] = (T)(f[e] * rs * (float)gam.e[e] + (float)bet.e[e]);
            }
            *reinterpret_cast<Vec16<T>*>(sa + (r0 + RPP * i) * WS_AP + c8 * 16) = x;
            if (rm && c8 == 0) s_mask[buf * WS_BM + r0 + RPP * i] = (float)pm[i];
        }
    };

    const int nslabs = (M + WS_BM - 1) / WS_BM;
    int slab = blockIdx.x;                               // grid <= nslabs
    const int pb_tile = PB ? args.plan.bias_tile : -1;
    fetch(slab, 0);                                      // the first slab travels while the weights are fetched
    // ---- weights: every wave reads the 32 rows of its slots as whole lines (a lane's fragments are 16-byte pieces
    // 32 bytes apart in one row, 32 rows per request: fetched that way every request touches 32 lines and uses a
    // quarter of each, and a workgroup's 128 .. 256 KB of weights do not stay in the first-level cache between the
    // K steps) and re-orders them through a private piece of the slab buffer, which is idle until the first commit.
    // A piece is 32 rows x PW channels; its 16-byte chunks are stored at chunk ^ (row % LR) so that the fragment
    // reads (one row per lane) spread over the banks.
    {
        constexpr int PW = WS_K < 128 ? WS_K : 128;      // channels per piece
        constexpr int LR = PW / 8;                       // 16-byte chunks (lanes) per row of a piece
        constexpr int NI = 32 / (64 / LR);               // requests per piece = K steps per piece
        constexpr int NP = WS_K / PW;                    // pieces per slot
        static_assert(NI * NP == WS_KS, "piece geometry");
        static_assert(WS_WAVES * 32 * PW * 2 <= 2 * WS_BM * WS_AP, "the staging area is the slab buffer");
        unsigned char* stage = s_a + wave * (32 * PW * 2);
        const int lrow = lane / LR, lcol = lane % LR;
#pragma unroll
        for (int sl = 0; sl < NS; ++sl)
#pragma unroll
            for (int pc = 0; pc < NP; ++pc)
#pragma unroll
                for (int i = 0; i < NI; ++i)
                    wf[sl][pc * NI + i] = MM::ld(W + (long)(s_wrow[sl] + i * (64 / LR) + lrow) * WS_K + pc * PW + lcol * 8);
        // tables the epilogues and the commits read from LDS (no global loads there); the barrier in front of the first
        // commit publishes them
        for (int i = tid; i < d.n_tiles * 128; i += WS_THREADS) {
            const ffk_tile& tb = d.tiles[i >> 7];
            const T* bp = (const T*)tb.bias;
            // gate halves of a GLU unit ([p 32 | g 32 | p 32 | g 32]) and sigmoid tiles: pre-multiplied for ws_sigmoid_pre
            const bool sig = tb.glu ? ((i >> 5) & 1) != 0 : tb.act == FFK_ACT_SIGMOID;
            const float b = bp ? (float)bp[i & 127] : 0.0f;
            s_bias[i] = sig ? -1.4426950408889634f * b : b;
        }

        {
            if (folded) {
                for (int i = tid; i < d.n_tiles * 128; i += WS_THREADS) s_c1[i] = ((const float*)d.ln_gamma)[i];
            }
            if (ln && !CM && tid < WS_K) {
                s_ln1[tid] = ((const T*)d.ln_gamma)[tid];
                s_ln1[WS_K + tid] = ((const T*)d.ln_beta)[tid];
            }
            if (ln && CM && tid < WS_K) {
                s_cmln[tid] = (float)((const T*)d.ln_gamma)[tid];
                s_cmln[WS_K + tid] = (float)((const T*)d.ln_beta)[tid];
            }
        }
        if (PB && pb_tile >= 0) {
            const int heads = d.tiles[pb_tile].ncols;
            for (int i = tid; i < 4 * WS_K; i += WS_THREADS)
                s_wb[i] = (i / WS_K) < heads ? W[(long)(pb_tile * 128 + i / WS_K) * WS_K + (i % WS_K)] : (T)0.0f;
        }
#pragma unroll
        for (int sl = 0; sl < NS; ++sl)
#pragma unroll
            for (int pc = 0; pc < NP; ++pc) {
#pragma unroll
                for (int i = 0; i < NI; ++i) {
                    const int row = i * (64 / LR) + lrow;
                    *reinterpret_cast<bf16x8*>(stage + row * (PW * 2) + ((lcol ^ (row & (LR - 1))) * 16)) = wf[sl][pc * NI + i];
                }
#pragma unroll
                for (int k = 0; k < NI; ++k)
                    wf[sl][pc * NI + k] = *reinterpret_cast<const bf16x8*>(
                        stage + s_wl[sl] * (PW * 2) + (((2 * k + half) ^ (s_wl[sl] & (LR - 1))) * 16));
            }
    }
    lds_barrier();                                       // every wave is done with the staging area
    commit(0);
    lds_barrier();
    int buf = 0;
    for (; slab < nslabs; slab += gridDim.x) {
        const bool more = slab + (int)gridDim.x < nslabs;
        if (more) fetch(slab + (int)gridDim.x, buf ^ 1);  // in flight during the products below
        const unsigned char* sa = s_a + buf * (WS_BM * WS_AP);
        if (PB && pb_tile >= 0) {
            // pair bias of this slab on the matrix pipe: wave w takes the rows 16 w .. 16 w + 15 as the N operand of
            // four 16 x 16 x 32 products against the (at most four) head weight rows, zero rows up to 16 (M operand).
            // The rows are the operand as the other products see it (normalised, rounded to bf16), so the value
            // equals a further output column group of four channels.  Result layout: lane = row, register v = head
            // (4 * (lane / 16) + v: only the first sixteen lanes hold real heads).
            const ffk_tile& tb = d.tiles[pb_tile];
            const int r16 = lane & 15, kq = lane >> 4;
            const unsigned char* xr = sa + (wave * 16 + r16) * WS_AP + kq * 16;
            const T* wr = s_wb + (r16 & 3) * WS_K + kq * 8;
            f32x4 pacc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int ks = 0; ks < WS_K / 32; ++ks) {
                const bf16x8 xv = *reinterpret_cast<const bf16x8*>(xr + ks * 64);
                bf16x8 wv = *reinterpret_cast<const bf16x8*>(wr + ks * 32);
                if (r16 >= 4) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) wv[e] = (T)0.0f;
                }
                pacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv, xv, pacc, 0, 0, 0);
            }
            const long pm = (long)slab * WS_BM + wave * 16 + r16;
            if (kq == 0 && pm < M) {
                const unsigned hi = (unsigned)pm / (unsigned)tb.inner, lo = (unsigned)pm - hi * (unsigned)tb.inner;
                T* po = (T*)tb.out + (long)(hi >> 5) * tb.s_o + (long)(lo >> 5) * 1024 + qk_tile_off((int)(lo & 31), (int)(hi & 31));
#pragma unroll
                for (int hd = 0; hd < 4; ++hd)
                    if (hd < tb.ncols) po[(long)hd * tb.s_h] = (T)(pacc[hd] * tb.scale);
            }
        }
        for (int rg = rg_first; rg < WS_RG; rg += rg_step) {
            const long m0g = (long)slab * WS_BM + rg * 32;
            if (m0g >= M) break;
            const unsigned char* ap = sa + (rg * 32 + n32) * WS_AP + half * 16;
            // position of this lane's row for the [row][channel] tiles; the division is redone only
            // when a slot's tile has another `inner`
            const long mrow = m0g + n32;
            const bool valid = mrow < M;
            const unsigned mc = (unsigned)(valid ? mrow : M - 1);
            unsigned c_inner = 0, c_hi = 0, c_lo = mc;
            const float* smk = s_mask + buf * WS_BM + rg * 32;
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                if (s_tile[s] < 0 || s_glu[s] == 2) continue;
                const WsSlot& t = sp[s];
                const bool glu = s_glu[s] == 1;
                const int sg = s + 1 < NS ? s + 1 : s;             // gate slot of a GLU unit (constant after unrolling)
                const float* sb = s_bias + s_wrow[s];
                // The A fragments are re-read from LDS for every slot: keeping them across the epilogue of
                // the previous slot costs 32 registers, and a single spilled register puts a scratch
                // reload with a full vector-memory wait into every epilogue.
                int reread = 0;
                asm volatile("" : "+v"(reread));                   // opaque zero: keeps the compiler from reusing the loads
                if constexpr (LEAN) {
                    const bool rows = by_rows[s];
                    // One straight-line body per (store order, GLU or not): the gate accumulator only exists
                    // where it is used, and no accumulator has to be copied or cleared where paths would join.
                    auto slot_body = [&](auto rows_tag, auto glu_tag) {
                        constexpr bool ROWS = decltype(rows_tag)::value, G = decltype(glu_tag)::value;
                        f32x16 acc, accg;
#pragma unroll
                        for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
                        if (G) {
#pragma unroll
                            for (int v = 0; v < 16; ++v) accg[v] = 0.0f;
                        }
                        if (DUAL && G) {
                            // gate half: fragments of the second operand's row (row % 16 == l32 % 16 picks the swizzle)
                            const unsigned a2row = (unsigned)(buf * (WS_BM * 256) + (rg * 32 + n32) * 256 + ((half ^ (n32 & 15)) << 4));
#pragma unroll
                            for (int k0 = 0; k0 < WS_KS; k0 += AFC) {
                                bf16x8 af[AFC];
#pragma unroll
                                for (int ks = 0; ks < AFC; ++ks)
                                    af[ks] = *reinterpret_cast<const bf16x8*>(s_a2 + ((a2row + reread) ^ (unsigned)((k0 + ks) * 32)));
#pragma unroll
                                for (int ks = 0; ks < AFC; ++ks) MM::mma(accg, wf[sg][k0 + ks], af[ks]);
                            }
                        }
#pragma unroll
                        for (int k0 = 0; k0 < WS_KS; k0 += AFC) {          // AFC K steps of A in registers at a time
                            bf16x8 af[AFC];
#pragma unroll
                            for (int ks = 0; ks < AFC; ++ks) af[ks] = *reinterpret_cast<const bf16x8*>(ap + reread + (k0 + ks) * 32);
                            if (ROWS) {
#pragma unroll
                                for (int ks = 0; ks < AFC; ++ks) MM::mma(acc, wf[s][k0 + ks], af[ks]);
                                if (!DUAL && G) {
#pragma unroll
                                    for (int ks = 0; ks < AFC; ++ks) MM::mma(accg, wf[sg][k0 + ks], af[ks]);
                                }
                            } else {
#pragma unroll
                                for (int ks = 0; ks < AFC; ++ks) MM::mma(acc, af[ks], wf[s][k0 + ks]);
                                if (G) {
#pragma unroll
                                    for (int ks = 0; ks < AFC; ++ks) MM::mma(accg, af[ks], wf[sg][k0 + ks]);
                                }
                            }
                        }
                        if (ROWS) {
                            if (t.inner != c_inner) {
                                c_inner = t.inner;
                                if (c_inner < (unsigned)M) {
                                    c_hi = mc / c_inner;
                                    c_lo = mc - c_hi * c_inner;
                                } else {
                                    c_hi = 0;
                                    c_lo = mc;
                                }
                            }
                            const float rmask = t.masked ? smk[n32] : 1.0f;
                            ws_store_rows<G, XT>(t, acc, G ? accg : acc, sb, valid, mc, c_hi, c_lo, rmask, half);
                        } else {
                            const float* sm = t.masked ? smk : nullptr;
                            ws_store_cols<G>(t, acc, G ? accg : acc, sb, sm, m0g, M, l32, half);
                        }
                    };
                    typedef std::integral_constant<bool, true> Yes;
                    typedef std::integral_constant<bool, false> No;
                    if (ALLOW_GLU && glu) {
                        if (rows) slot_body(Yes(), Yes());
                        else slot_body(No(), Yes());
                    } else {
                        if (rows) slot_body(Yes(), No());
                        else slot_body(No(), No());
                    }
                } else {
                    f32x16 acc, accg;
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[v] = accg[v] = 0.0f;
                    float st1 = 0.0f, st2 = 0.0f, su1 = 0.0f, su2 = 0.0f;   // row statistics of the two operands (DUAL)
                    const bool rows = by_rows[s];
                    if (DUAL && ALLOW_GLU && glu) {
                        // gate half: fragments of the second operand's row (row % 16 == l32 % 16 picks the swizzle)
                        const unsigned a2row = (unsigned)(buf * (WS_BM * 256) + (rg * 32 + n32) * 256 + ((half ^ (n32 & 15)) << 4));
#pragma unroll
                        for (int k0 = 0; k0 < WS_KS; k0 += AFC) {
                            bf16x8 af[AFC];
#pragma unroll
                            for (int ks = 0; ks < AFC; ++ks)
                                af[ks] = *reinterpret_cast<const bf16x8*>(s_a2 + ((a2row + reread) ^ (unsigned)((k0 + ks) * 32)));
                            {
                                typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
                                const bf16x2 ones = {(bf16_t)1.0f, (bf16_t)1.0f};
#pragma unroll
                                for (int ks = 0; ks < AFC; ++ks)
#pragma unroll
                                    for (int e = 0; e < 4; ++e) {
                                        const bf16x2 pr = {af[ks][2 * e], af[ks][2 * e + 1]};
                                        su1 = __builtin_amdgcn_fdot2_f32_bf16(pr, ones, su1, false);
                                        su2 = __builtin_amdgcn_fdot2_f32_bf16(pr, pr, su2, false);
                                    }
                            }
#pragma unroll
                            for (int ks = 0; ks < AFC; ++ks) MM::mma(accg, wf[sg][k0 + ks], af[ks]);
                        }
                    }
#pragma unroll
                    for (int k0 = 0; k0 < WS_KS; k0 += AFC) {          // AFC K steps of A in registers at a time
                        bf16x8 af[AFC];
#pragma unroll
                        for (int ks = 0; ks < AFC; ++ks) af[ks] = *reinterpret_cast<const bf16x8*>(ap + reread + (k0 + ks) * 32);
                        if (DUAL && folded) {
                            // sum and sum of squares of this lane's half of its row, from the fragments themselves
                            typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
                            const bf16x2 ones = {(bf16_t)1.0f, (bf16_t)1.0f};
#pragma unroll
                            for (int ks = 0; ks < AFC; ++ks)
#pragma unroll
                                for (int e = 0; e < 4; ++e) {
                                    const bf16x2 pr = {af[ks][2 * e], af[ks][2 * e + 1]};
                                    st1 = __builtin_amdgcn_fdot2_f32_bf16(pr, ones, st1, false);
                                    st2 = __builtin_amdgcn_fdot2_f32_bf16(pr, pr, st2, false);
                                }
                        }
                        if (rows) {
#pragma unroll
                            for (int ks = 0; ks < AFC; ++ks) MM::mma(acc, wf[s][k0 + ks], af[ks]);
                            if (!DUAL && ALLOW_GLU && glu) {
#pragma unroll
                                for (int ks = 0; ks < AFC; ++ks) MM::mma(accg, wf[sg][k0 + ks], af[ks]);
                            }
                        } else {
#pragma unroll
                            for (int ks = 0; ks < AFC; ++ks) MM::mma(acc, af[ks], wf[s][k0 + ks]);
                            if (ALLOW_GLU && glu) {
#pragma unroll
                                for (int ks = 0; ks < AFC; ++ks) MM::mma(accg, af[ks], wf[sg][k0 + ks]);
                            }
                        }
                    }
                    if (rows) {
                        if (t.inner != c_inner) {
                            c_inner = t.inner;
                            if (c_inner < (unsigned)M) {
                                c_hi = mc / c_inner;
                                c_lo = mc - c_hi * c_inner;
                            } else {
                                c_hi = 0;
                                c_lo = mc;
                            }
                        }
                        const float rmask = t.masked ? smk[n32] : 1.0f;
                        if (DUAL && folded) {
                            st1 += lane_xor<32>(st1);
                            st2 += lane_xor<32>(st2);
                            const float mean = st1 * (1.0f / WS_K);
                            const float rstd = rsqrtf(fmaxf(st2 * (1.0f / WS_K) - mean * mean, 0.0f) + d.ln_eps);
                            su1 += lane_xor<32>(su1);
                            su2 += lane_xor<32>(su2);
                            const float mean_g = su1 * (1.0f / WS_K);
                            const float rstd_g = -1.4426950408889634f * rsqrtf(fmaxf(su2 * (1.0f / WS_K) - mean_g * mean_g, 0.0f) + d.ln_eps);
                            const unsigned char* a2r = nullptr;
                            int a2v = 0;
                            if (args.plan.resid_a2 && t.resid) {
                                a2r = s_a2 + buf * (WS_BM * 256) + (rg * 32 + n32) * 256;
                                a2v = (int)(t.resid - (const T*)d.a2) / 8 + 2 * half;
                            }
                            ws_store_rows_folded<XT>(t, acc, accg, sb, s_c1 + s_wrow[s], rstd, -rstd * mean, rstd_g, -rstd_g * mean_g,
                                                 valid, c_hi, c_lo, half, a2r, a2v, n32 & 15);
                        } else if (ALLOW_GLU && glu) ws_store_rows_compact<true, XT>(t, acc, accg, sb, valid, mc, c_hi, c_lo, rmask, half);
                        else ws_store_rows_compact<false, XT>(t, acc, accg, sb, valid, mc, c_hi, c_lo, rmask, half);
                    } else {
                        const float* sm = t.masked ? smk : nullptr;
                        if (ALLOW_GLU && glu) ws_store_cols_compact<true>(t, acc, accg, sb, sm, m0g, M, l32, half);
                        else ws_store_cols_compact<false>(t, acc, accg, sb, sm, m0g, M, l32, half);
                    }
                }
            }
        }
        if (!more) break;                                // nothing left to commit: the stores drain on their own
        commit(buf ^ 1);
        lds_barrier();
        buf ^= 1;
    }
}

// tiles stored with channels contiguous (lane = row) vs rows contiguous (lane = channel): host side
bool ws_tile_ok(const ffk_linear_desc& d, const ffk_tile& t) {
    auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    if (t.inner <= 0 || t.ncols <= 0 || !al16(t.out)) return false;
    if (ws_by_rows(t)) {
        if (t.kind == FFK_TILE_STRIDED) {
            if (t.ncols % 8 != 0 || t.s_o % 8 || t.s_i % 8 || t.s_h % 8) return false;
            if (t.resid && !al16(t.resid)) return false;
            if (t.gate && (!al16(t.gate) || t.gate_ld % 8)) return false;
            if (t.xtail && (!t.resid || t.ncols % 16 != 0 || t.s_o % 16 || t.s_i % 16 || t.s_h % 16)) return false;
        } else {
            if (t.ncols % 32 != 0 || t.resid || t.gate || t.xtail || t.s_o % 8 || t.s_h % 8) return false;
        }
        return true;
    }
    if (t.resid || t.gate || t.xtail) return false;
    if (t.kind == FFK_TILE_V) return t.inner % 32 == 0 && t.ncols % 32 == 0 && t.s_o % 8 == 0 && t.s_h % 8 == 0;
    if (t.kind != FFK_TILE_STRIDED) return false;
    return d.M % 16 == 0 && t.inner % 16 == 0 && t.s_i == 1 && t.s_o % 8 == 0 && t.s_h % 8 == 0 && t.s_d % 8 == 0;
}

// Distributes the 32-row weight units over the waves.  The waves form G = 8 / R groups; the R waves
// of a group hold the same units and take every R-th row group of a slab (R as large as the units
// allow, so that few units still use all eight waves).  Returns false if the units do not fit.
bool ws_make_plan(const ffk_linear_desc& d, WsPlan& p, int rg_per_slab, int max_ns) {
    struct Unit { int tile, chan, wrow, slots; };
    Unit units[FFK_MAX_TILES * 4];
    int nu = 0;
    for (int i = 0; i < d.n_tiles; ++i) {
        const ffk_tile& t = d.tiles[i];
        const int n = (t.ncols + 31) / 32;
        for (int u = 0; u < n; ++u) {
            Unit x;
            x.tile = i;
            x.chan = u * 32;
            x.wrow = i * 128 + (t.glu ? u * 64 : u * 32);
            x.slots = t.glu ? 2 : 1;
            units[nu++] = x;
        }
    }
    int assign[WS_WAVES][WS_NS];
    int G = 0, R = 0;
    for (R = rg_per_slab; R >= 1; R >>= 1) {
        G = WS_WAVES / R;
        int load[WS_WAVES] = {0};
        for (int g = 0; g < G; ++g)
            for (int s = 0; s < WS_NS; ++s) assign[g][s] = -1;
        bool fits = true;
        for (int pass = 2; pass >= 1 && fits; --pass) {            // two-slot (GLU) units first
            for (int i = 0; i < nu && fits; ++i) {
                if (units[i].slots != pass) continue;
                int best = -1;
                for (int g = 0; g < G; ++g)
                    if (load[g] + pass <= max_ns && (best < 0 || load[g] < load[best])) best = g;
                if (best < 0) {
                    fits = false;
                    break;
                }
                assign[best][load[best]] = i;
                if (pass == 2) assign[best][load[best] + 1] = -2 - i;   // gate half of unit i
                load[best] += pass;
            }
        }
        if (fits) break;
    }
    if (R < 1) return false;
    p.max_slots = 0;
    for (int g = 0; g < G; ++g) {
        int n = 0;
        for (int sl = 0; sl < WS_NS; ++sl) n += assign[g][sl] != -1;
        p.max_slots = n > p.max_slots ? n : p.max_slots;
    }
    for (int w = 0; w < WS_WAVES; ++w) {
        const int g = w % G;
        p.rg_first[w] = w / G;
        p.rg_step[w] = R;
        for (int s = 0; s < WS_NS; ++s) {
            const int a = assign[g][s];
            if (a == -1) {
                p.tile[w][s] = -1;
                p.wrow[w][s] = p.chan[w][s] = p.glu[w][s] = 0;
            } else if (a >= 0) {
                p.tile[w][s] = units[a].tile;
                p.wrow[w][s] = units[a].wrow;
                p.chan[w][s] = units[a].chan;
                p.glu[w][s] = units[a].slots == 2 ? 1 : 0;
            } else {
                const Unit& u = units[-2 - a];
                p.tile[w][s] = u.tile;
                p.wrow[w][s] = u.wrow + 32;
                p.chan[w][s] = u.chan;
                p.glu[w][s] = 2;
            }
        }
    }
    return true;
}

template <int NS, int K, bool CM, bool DUAL = false, bool XT = false>
int ws_launch(const WsArgs& args, hipStream_t st) {
    constexpr int WS_BM = WsGeo<K>::BM;
    const size_t smem = 2 * (size_t)WS_BM * WsGeo<K>::AP + 2 * WS_BM * sizeof(float) + FFK_MAX_TILES * 128 * sizeof(float) +
                        (DUAL ? 2 * (size_t)WS_BM * 256 + 256 * sizeof(T) + FFK_MAX_TILES * 128 * sizeof(float) : 0) +
                        (CM ? 256 * sizeof(float) : 2 * K * sizeof(T)) +
                        (!CM && !DUAL && !XT && K == 128 ? 4 * K * sizeof(T) : 0);      // head weights of a pair-bias tile
    static FfkLdsReservation lds_reserved;
    {
        const int rc_lds = ffk_reserve_lds(lds_reserved, (const void*)linear_ws_kernel<NS, K, CM, DUAL, XT>, smem, "ffk_fused_linear");
        if (rc_lds != FFK_OK) return rc_lds;
    }
    const int nslabs = ffk_cdiv(args.d.M, WS_BM);
    const int grid = nslabs < WS_MAX_GRID ? nslabs : WS_MAX_GRID;
    linear_ws_kernel<NS, K, CM, DUAL, XT><<<grid, WS_THREADS, smem, st>>>(args);
    return ffk_check_launch("ffk_fused_linear");
}

}  // namespace

// Launches the weights-stationary kernel if it can take this (already validated) descriptor and
// returns 1 with the launch status in *status; returns 0 if the caller has to use another variant.
int ffk_linear_ws_try(const ffk_linear_desc* d, hipStream_t st, int* status) {
    if (d->dtype != FFK_BF16 || (d->K != 64 && d->K != 128 && d->K != 256)) return 0;
    if ((d->ln_folded != 0) != (d->a2 != nullptr)) return 0;    // folded LayerNorms and the second operand go together
    if (d->a_chanmajor && ((d->K != 128 && d->K != 64) || d->a_si != 1 || d->a_inner % 8 || d->a_so % 8 || d->a_cs % 8 || d->M % 8)) return 0;
    if (d->a2 && d->K != 128) return 0;                          // the second operand is built for K = 128
    const bool k256 = d->K == 256;
    if (d->variant == FFK_LINEAR_STAGED) return 0;
    bool chan_major = false, v_tiles = false, tails = false;
    int mask_tile = -1;
    // a trailing pair-bias tile (score-operand tiles of <= 4 heads) rides on the launch without a weight slot
    int n_slot_tiles = d->n_tiles, bias_tile = -1;
    if (d->n_tiles >= 2 && d->tiles[d->n_tiles - 1].kind == FFK_TILE_BIAS) {
        const ffk_tile& t = d->tiles[d->n_tiles - 1];
        auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
        if (d->K != 128 || d->a_chanmajor || d->a2 || t.ncols < 1 || t.ncols > 4 || t.bias || t.resid || t.gate || t.rowmask ||
            t.xtail || t.glu || t.act != FFK_ACT_NONE || t.inner <= 0 || !t.out || !al16(t.out))
            return 0;
        bias_tile = d->n_tiles - 1;
        n_slot_tiles = d->n_tiles - 1;
    }
    for (int i = 0; i < n_slot_tiles; ++i) {
        const ffk_tile& t = d->tiles[i];
        if (t.kind == FFK_TILE_BIAS) return 0;
        if (!ws_tile_ok(*d, t)) return 0;
        tails = tails || t.xtail != nullptr;
        chan_major = chan_major || (!ws_by_rows(t) && t.kind == FFK_TILE_STRIDED);
        v_tiles = v_tiles || t.kind == FFK_TILE_V;
        if (t.rowmask) {
            if (mask_tile < 0) {
                mask_tile = i;
            } else {
                const ffk_tile& f = d->tiles[mask_tile];     // one mask per launch
                if (t.rowmask != f.rowmask || t.inner != f.inner || t.m_so != f.m_so || t.m_si != f.m_si) return 0;
            }
        }
    }
    if (chan_major && v_tiles) return 0;          // they need different row orders within a group
    WsArgs args;
    const bool k64 = d->K == 64;
    {
        ffk_linear_desc slots = *d;                   // the plan covers the tiles that take weight slots
        slots.n_tiles = n_slot_tiles;
        if (!ws_make_plan(slots, args.plan, k256 ? WsGeo<256>::RG : (k64 ? WsGeo<64>::RG : WsGeo<128>::RG),
                          k256 ? 2 : (k64 ? 4 : 3)))
            return 0;
    }
    if (bias_tile >= 0 && (tails || chan_major)) return 0;   // built into the plain K = 128 variants only
    if (k256) {
        for (int i = 0; i < d->n_tiles; ++i)
            if (d->tiles[i].glu) return 0;                   // GLU units are only built for K = 128
    }
    args.plan.row_perm = chan_major ? 1 : 0;
    args.plan.mask_tile = mask_tile;
    args.plan.resid_a2 = 0;
    args.plan.bias_tile = bias_tile;
    args.d = *d;
    if (d->a2) {
        // second operand: every unit must be a GLU unit stored [row][channel], first operand channel-major
        if (!d->a_chanmajor || args.plan.max_slots > 2 || mask_tile >= 0 || d->a2_si % 8 || d->a2_so % 8) return 0;
        bool resid_a2 = true;
        for (int i = 0; i < d->n_tiles; ++i) {
            const ffk_tile& t = d->tiles[i];
            if (!t.glu || !ws_by_rows(t)) return 0;
            // plain residual GLU tiles of 64 channels only
            if (t.kind != FFK_TILE_STRIDED || t.gate || t.rowmask || t.scale != 1.0f || t.ncols != 64) return 0;
            // the residual is the second operand itself: same rows, channels [c0, c0 + 64) of its 128
            const long c0 = (const T*)t.resid - (const T*)d->a2;
            if (!t.resid || c0 < 0 || c0 + t.ncols > 128 || c0 % 32 || t.s_o != d->a2_so || t.s_i != d->a2_si ||
                t.inner != d->a2_inner || t.s_h != 32 || t.s_d != 1)
                resid_a2 = false;
        }
        args.plan.resid_a2 = resid_a2 ? 1 : 0;
        *status = tails ? ws_launch<2, 128, true, true, true>(args, st) : ws_launch<2, 128, true, true>(args, st);
    } else if (tails) {
        // residual tails: built for the output projections of the attentions (one plain tile group, two slots)
        if (d->a_chanmajor || args.plan.max_slots > 2 || k64) return 0;
        *status = k256 ? ws_launch<2, 256, false, false, true>(args, st) : ws_launch<2, 128, false, false, true>(args, st);
    } else if (d->a_chanmajor) {
        if (args.plan.max_slots > 2 || mask_tile >= 0) return 0;
        *status = k64 ? ws_launch<2, 64, true>(args, st) : ws_launch<2, 128, true>(args, st);
    } else if (k256) {
        *status = ws_launch<2, 256, false>(args, st);
    } else if (k64) {
        *status = args.plan.max_slots <= 2 ? ws_launch<2, 64, false>(args, st) : ws_launch<4, 64, false>(args, st);
    } else {
        *status = args.plan.max_slots <= 2 ? ws_launch<2, 128, false>(args, st) : ws_launch<3, 128, false>(args, st);
    }
    return 1;
}
