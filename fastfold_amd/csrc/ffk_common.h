// Shared device/host helpers for the ffk kernel library (gfx950 / CDNA4 only).
//
// Everything here is header-only: dtype traits, 16-byte vector access, wave-level
// reductions (64-wide wavefronts), MFMA fragment wrappers and the error plumbing
// behind the C ABI declared in include/ffk.h.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <atomic>
#include <mutex>

#include "../../include/ffk.h"

// ---------------------------------------------------------------- errors ----
extern thread_local char ffk_err_buf[512];
int ffk_fail(int code, const char* fmt, ...);

#define FFK_REQUIRE(cond, code, ...)                  \
    do {                                              \
        if (!(cond)) return ffk_fail((code), __VA_ARGS__); \
    } while (0)

int ffk_linear_slab_launch(const ffk_linear_desc* d, hipStream_t st);   // ffk_linear_slab.hip
int ffk_bgemm_big_try(const ffk_bgemm_desc* d, hipStream_t st, int* status);    // ffk_bgemm_big.hip
int ffk_linear_ws_try(const ffk_linear_desc* d, hipStream_t st, int* status);   // ffk_linear_ws.hip

// Dynamic-LDS reservation of one kernel: hipFuncSetAttribute is needed once per device (again only if a
// later launch asks for more).  A function-scope `static FfkLdsReservation` (zero-initialised) remembers, per
// device, what has been reserved; the slow path is serialised so that concurrent first calls from several host
// threads cannot leave a smaller reservation behind than the one recorded.
constexpr int FFK_MAX_DEVICES = 64;
struct FfkLdsReservation {
    std::atomic<size_t> bytes[FFK_MAX_DEVICES];
};
std::mutex& ffk_config_mutex();    // ffk_rowops.hip
static inline int ffk_reserve_lds(FfkLdsReservation& r, const void* func, size_t smem, const char* what) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return ffk_fail(FFK_ERR_LAUNCH, "%s: hipGetDevice: %s", what, hipGetErrorString(e));
    if (dev < 0 || dev >= FFK_MAX_DEVICES) return ffk_fail(FFK_ERR_UNSUPPORTED, "%s: device ordinal %d not supported", what, dev);
    if (smem <= r.bytes[dev].load(std::memory_order_acquire)) return FFK_OK;
    std::lock_guard<std::mutex> lock(ffk_config_mutex());
    if (smem <= r.bytes[dev].load(std::memory_order_relaxed)) return FFK_OK;
    e = hipFuncSetAttribute(func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return ffk_fail(FFK_ERR_LAUNCH, "%s: cannot reserve %zu B of LDS: %s", what, smem, hipGetErrorString(e));
    r.bytes[dev].store(smem, std::memory_order_release);
    return FFK_OK;
}

static inline bool ffk_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Checks the launch that was just issued on this thread.
static inline int ffk_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return ffk_fail(FFK_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return FFK_OK;
}

// ---------------------------------------------------------------- dtypes ----
typedef __bf16 bf16_t;
typedef _Float16 f16_t;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename T> struct DT;
template <> struct DT<float> {
    static constexpr int VEC = 4;      // elements per 16-byte vector
    static __device__ __forceinline__ float to_f(float v) { return v; }
    static __device__ __forceinline__ float from_f(float v) { return v; }
};
template <> struct DT<bf16_t> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ float to_f(bf16_t v) { return (float)v; }
    static __device__ __forceinline__ bf16_t from_f(float v) { return (bf16_t)v; }
};
template <> struct DT<f16_t> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ float to_f(f16_t v) { return (float)v; }
    static __device__ __forceinline__ f16_t from_f(float v) { return (f16_t)v; }
};

// 16 bytes of T, loaded/stored as one dwordx4 access.
template <typename T> struct alignas(16) Vec16 {
    T e[DT<T>::VEC];
};

template <typename T> __device__ __forceinline__ Vec16<T> ld16(const T* p) {
    return *reinterpret_cast<const Vec16<T>*>(p);
}
template <typename T> __device__ __forceinline__ void st16(T* p, const Vec16<T>& v) {
    *reinterpret_cast<Vec16<T>*>(p) = v;
}
// Streaming (non-temporal) variants for data that is touched exactly once.
template <typename T> __device__ __forceinline__ Vec16<T> ld16_nt(const T* p) {
    u32x4 r = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return *reinterpret_cast<Vec16<T>*>(&r);
}
template <typename T> __device__ __forceinline__ void st16_nt(T* p, const Vec16<T>& v) {
    __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(&v), reinterpret_cast<u32x4*>(p));
}

// ------------------------------------------------------- wave reductions ----
// lane_xor<W>(v): the value of lane (l ^ W) for a v that is already uniform over aligned groups of W
// lanes - which is all a butterfly reduction needs.  1 and 2 are quad permutes, 4 and 8 the half-row
// and row mirrors of the DPP unit (lane i reads lane 7 - i / 15 - i: another lane of the partner group,
// holding the same value as lane i ^ W), 16 and 32 the row / half-wave swap instructions.  None of them
// goes through the LDS crossbar, unlike a general shuffle.
template <int W> __device__ __forceinline__ float lane_xor(float v) {
    const int x = __builtin_bit_cast(int, v);
    int r;
    if (W == 1) r = __builtin_amdgcn_update_dpp(x, x, 0xB1, 0xF, 0xF, false);          // quad_perm [1,0,3,2]
    else if (W == 2) r = __builtin_amdgcn_update_dpp(x, x, 0x4E, 0xF, 0xF, false);     // quad_perm [2,3,0,1]
    else if (W == 4) r = __builtin_amdgcn_update_dpp(x, x, 0x141, 0xF, 0xF, false);    // row_half_mirror
    else if (W == 8) r = __builtin_amdgcn_update_dpp(x, x, 0x140, 0xF, 0xF, false);    // row_mirror
    else if (W == 16) {
        // a = b = v;  swap(a rows 1 / 3, b rows 0 / 2):  a = [r0 r0 r2 r2], b = [r1 r1 r3 r3]
        typedef unsigned u2 __attribute__((ext_vector_type(2)));
        const u2 p = __builtin_amdgcn_permlane16_swap((unsigned)x, (unsigned)x, false, false);
        const int lane_row = (__lane_id() >> 4) & 1;
        r = (int)(lane_row ? p[0] : p[1]);
    } else {
        typedef unsigned u2 __attribute__((ext_vector_type(2)));
        const u2 p = __builtin_amdgcn_permlane32_swap((unsigned)x, (unsigned)x, false, false);
        r = (int)((__lane_id() >> 5) ? p[0] : p[1]);
    }
    return __builtin_bit_cast(float, r);
}
// Reduce over groups of `width` adjacent lanes (width a power of two <= 64); every lane gets the result.
// The streaming row kernels, whose group size is a run-time value, measured faster with the general
// shuffles (softmax 59.5 vs 64 us) and keep them.
__device__ __forceinline__ float group_sum(float v, int width) {
    if (!__builtin_constant_p(width)) {     // group size only known at run time (the row kernels): general shuffles
        for (int off = width >> 1; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
        return v;
    }
    if (width >= 2) v += lane_xor<1>(v);
    if (width >= 4) v += lane_xor<2>(v);
    if (width >= 8) v += lane_xor<4>(v);
    if (width >= 16) v += lane_xor<8>(v);
    if (width >= 32) v += lane_xor<16>(v);
    if (width >= 64) v += lane_xor<32>(v);
    return v;
}
__device__ __forceinline__ float group_max(float v, int width) {
    if (!__builtin_constant_p(width)) {
        for (int off = width >> 1; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
        return v;
    }
    if (width >= 2) v = fmaxf(v, lane_xor<1>(v));
    if (width >= 4) v = fmaxf(v, lane_xor<2>(v));
    if (width >= 8) v = fmaxf(v, lane_xor<4>(v));
    if (width >= 16) v = fmaxf(v, lane_xor<8>(v));
    if (width >= 32) v = fmaxf(v, lane_xor<16>(v));
    if (width >= 64) v = fmaxf(v, lane_xor<32>(v));
    return v;
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every
// outstanding global load / store of the wave (vmcnt(0)), which would serialise the register
// prefetches and the fire-and-forget output stores of the streaming kernels with each barrier.
// No kernel here communicates between waves through global memory, so LDS ordering suffices.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ------------------------------------------------------------ fast math ----
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
// max(x, 0) in one instruction: fmaxf first canonicalises its argument (a second v_max) under IEEE rules
__device__ __forceinline__ float relu_f(float x) { return __builtin_amdgcn_fmed3f(x, 0.0f, 3.0e38f); }
__device__ __forceinline__ float sigmoid_f(float x) {
    // 1 / (1 + 2^(-x*log2e))
    return fast_rcp(1.0f + fast_exp2(-1.4426950408889634f * x));
}
template <typename T> __device__ __forceinline__ float exp_for(float x);
template <> __device__ __forceinline__ float exp_for<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ float exp_for<bf16_t>(float x) { return fast_exp2(1.4426950408889634f * x); }
template <> __device__ __forceinline__ float exp_for<f16_t>(float x) { return fast_exp2(1.4426950408889634f * x); }

// ------------------------------------------------- extended residual stream ----
// A residual stream that is rounded to bf16 after every one of the ~300 updates of a 48-block stack drifts by
// a random walk of half-ulp errors (about 2e-2 relative at the end).  The stream can therefore carry eight more
// mantissa bits in a separate byte tensor ("tail", same element addressing as the bf16 tensor): the pair (h, t)
// stands for the fp32 bit pattern (bits(h) << 16) + (t << 8), t a signed byte.  h is the value rounded to bf16
// (half up, after rounding to 24 bits), so every reader that ignores the tail still sees a correctly rounded
// bf16 tensor; only the kernels that add an update to the stream read and rewrite the tail.  Every such epilogue
// rounds its update to bf16 first and then adds it at 24 bits, so that kernel variants (and chunked runs, which
// may pick another variant for a ragged piece) agree bit for bit.
__device__ __forceinline__ float xs_value(bf16_t h, int8_t t) {
    const uint32_t hw = (uint32_t)__builtin_bit_cast(uint16_t, h) << 16;
    return __builtin_bit_cast(float, hw + ((uint32_t)(int32_t)t << 8));
}
__device__ __forceinline__ void xs_round(float x, bf16_t* h, int8_t* t) {
    const uint32_t w24 = __builtin_bit_cast(uint32_t, x) + 0x80u;
    *h = __builtin_bit_cast(bf16_t, (uint16_t)((w24 + 0x8000u) >> 16));
    *t = (int8_t)(uint8_t)(w24 >> 8);
}
// Eight consecutive elements: hv holds the bf16 values, (t0, t1) their tails.
__device__ __forceinline__ void xs_decode8(const u32x4& hv, uint32_t t0, uint32_t t1, float* f) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t hw = (i & 1) ? (hv[i >> 1] & 0xFFFF0000u) : (hv[i >> 1] << 16);
        const int32_t t = __builtin_amdgcn_sbfe((int32_t)(i < 4 ? t0 : t1), 8 * (i & 3), 8);
        f[i] = __builtin_bit_cast(float, hw + ((uint32_t)t << 8));
    }
}
__device__ __forceinline__ void xs_encode8(const float* f, u32x4& hv, uint32_t& t0, uint32_t& t1) {
    uint32_t w[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = __builtin_bit_cast(uint32_t, f[i]) + 0x80u;
#pragma unroll
    for (int j = 0; j < 4; ++j)      // high halves of (w + 0x8000) of two neighbours
        hv[j] = __builtin_amdgcn_perm(w[2 * j + 1] + 0x8000u, w[2 * j] + 0x8000u, 0x07060302u);
    // byte 1 of four neighbours
    const uint32_t a = __builtin_amdgcn_perm(w[1], w[0], 0x0c0c0501u), b = __builtin_amdgcn_perm(w[3], w[2], 0x0c0c0501u);
    const uint32_t c = __builtin_amdgcn_perm(w[5], w[4], 0x0c0c0501u), e = __builtin_amdgcn_perm(w[7], w[6], 0x0c0c0501u);
    t0 = __builtin_amdgcn_perm(b, a, 0x05040100u);
    t1 = __builtin_amdgcn_perm(e, c, 0x05040100u);
}

__device__ __forceinline__ void xs_encode8(const float* f, u32x4& hv, u32x2& tn) {
    uint32_t a, b;
    xs_encode8(f, hv, a, b);
    tn[0] = a;
    tn[1] = b;
}
// Sixteen consecutive elements of a lane: (r0, r1) the stream's bf16 values, tv their tail bytes; the update is
// added to the 24-bit value and the result split again into (h0, h1) and tn.
__device__ __forceinline__ void xs_update16(const float* upd, const u32x4& r0, const u32x4& r1, const u32x4& tv, u32x4& h0,
                                            u32x4& h1, u32x4& tn) {
    float f[16];
    xs_decode8(r0, tv[0], tv[1], f);
    xs_decode8(r1, tv[2], tv[3], f + 8);
#pragma unroll
    for (int i = 0; i < 16; ++i) f[i] += upd[i];
    uint32_t a, b, c, e;
    xs_encode8(f, h0, a, b);
    xs_encode8(f + 8, h1, c, e);
    tn[0] = a;
    tn[1] = b;
    tn[2] = c;
    tn[3] = e;
}

// ----------------------------------------------------------------- MFMA ----
// A "fragment" is the 16 bytes one lane contributes to a 32x32 MFMA operand:
// lane l supplies row (l & 31) of the operand and K-group (l >> 5).  For bf16 the
// 16 bytes are 8 consecutive K elements and one v_mfma_f32_32x32x16_bf16 consumes
// the pair (K step 16).  For fp32 they are 4 consecutive K elements and four
// v_mfma_f32_32x32x2_f32 consume them (element t of both operands in step t), which
// covers K step 8.  Both operands must be fetched with the same K <-> slot mapping;
// the sum over K is then independent of that mapping.
//
// Accumulator layout (both dtypes): lane l holds column (l & 31) of the 32x32 tile;
// register v (0..15) holds row  8*(v/4) + 4*(l>>5) + (v%4).
template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
    static constexpr int KSTEP = 16;   // K elements consumed per fragment pair
    static constexpr int KLANE = 8;    // K elements per lane per fragment
    typedef bf16x8 Frag;
    static __device__ __forceinline__ void mma(f32x16& acc, const Frag& a, const Frag& b) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
    }
    static __device__ __forceinline__ Frag ld(const bf16_t* p) { return *reinterpret_cast<const Frag*>(p); }
};
template <> struct Mma<float> {
    static constexpr int KSTEP = 8;
    static constexpr int KLANE = 4;
    typedef f32x4 Frag;
    static __device__ __forceinline__ void mma(f32x16& acc, const Frag& a, const Frag& b) {
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], b[0], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[1], b[1], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[2], b[2], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[3], b[3], acc, 0, 0, 0);
    }
    static __device__ __forceinline__ Frag ld(const float* p) { return *reinterpret_cast<const Frag*>(p); }
};

// Row of the 32x32 accumulator tile held in register v by lane `lane`.
__device__ __forceinline__ int acc_row(int v, int lane) { return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3); }

static inline int ffk_cdiv(long a, long b) { return (int)((a + b - 1) / b); }

// ------------------------------------------------- attention operand tiles ----
// q / k, v and the additive bias are exchanged between the projection kernel and the
// attention kernel in 32x32-element tiles (1024 elements each) whose internal order is
// exactly what one wavefront loads as an MFMA operand / accumulator, so that every
// lane reads 16 contiguous elements and a wave reads the tile as one contiguous block.
//
//  q/k tile (rows n, head dim d):  lane (n%32, kg=d/16) owns d = 16*kg .. 16*kg+15
__host__ __device__ __forceinline__ int qk_tile_off(int n32, int d) { return (d >> 4) * 512 + n32 * 16 + (d & 15); }
//  accumulator-order tile: element (row, col) of a 32x32 tile whose column is the lane's
//  (l & 31) and whose rows are spread over (l >> 5, register) as in the MFMA accumulator:
//  lane = ((row & 7) >> 2) * 32 + col,  register = 4 * (row >> 3) + (row & 3).
//  Used for v (row = key, col = head-dim index).  The additive bias uses the q/k order with
//  rows = keys and the 32 queries of the tile in place of the head dim.
__host__ __device__ __forceinline__ int acc_tile_off(int row, int col) {
    return ((((row & 7) >> 2) * 32 + col) << 4) + 4 * (row >> 3) + (row & 3);
}
