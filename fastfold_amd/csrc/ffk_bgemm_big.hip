// Large-tile variant of the batched NT GEMM (see ffk_bgemm_nt in include/ffk.h) for bf16 with
// K % 32 == 0 and 16-byte aligned, channel-contiguous output.
//
// 512 threads = 8 wavefronts in a 4 x 2 grid.  Two shapes:
//   wide   256 x 256 block, 64 x 128 per wave (8 accumulator tiles): six LDS fragment reads feed eight
//          MFMAs per K step, which keeps the LDS below its bandwidth limit at full matrix rate
//          (the 64 x 64 wave tile of the small kernel needs four reads per four MFMAs and saturates it);
//   narrow 256 x 128 block, 64 x 64 per wave, for N <= 128 (projections; bound by reading A).
// The K loop moves 32-element chunks through a four-slot LDS ring that is filled by direct
// global -> LDS loads (no registers, no LDS stores): three chunks are in flight behind the one being
// multiplied, which is what covers the memory latency with a single workgroup per CU.  Rows are
// unpadded 64-byte lines; an XOR swizzle of their four 16-byte columns keeps the fragment reads free
// of bank conflicts.  All addresses are set up once per tile.
// A chunk holds two K steps of 16.  The steps are software-pipelined across the chunk barrier: the
// fragments of a chunk's second K step are read while its first K step is multiplied, and multiplied
// behind the next barrier while the next chunk's first fragments are on their way, so neither the
// barrier nor the LDS read latency leaves the matrix pipe without queued work.
// The MFMA computes C^T (rows of B are the M operand) and reads the B rows of a 32-row group through
// the permutation tau(8a + 4h + b) = 16h + 4a + b, so that a lane ends up with 16 consecutive
// output columns of one row: the epilogue (bias / activation / scale / row divisor / residual) works
// on registers and stores 32 contiguous bytes per lane, with no staging through LDS.
#include "ffk_common.h"
#include <stdlib.h>

namespace {

typedef bf16_t T;
constexpr int BG_THREADS = 512;
constexpr int BG_BK = 32;                    // K elements per chunk: 64-byte rows, four 16-byte columns
constexpr int BG_SLOTS = 4;                  // LDS ring depth: three chunks in flight behind the one in use

__device__ __forceinline__ int bg_tau(int i) { return ((i >> 2) & 1) * 16 + (i >> 3) * 4 + (i & 3); }

// One 16-byte column of a chunk row goes from global memory straight into LDS (no registers): the
// hardware places lane L of the wave at  dst + 16 * L,  dst being wave-uniform.
__device__ __forceinline__ void bg_load_lds(const T* src, unsigned char* dst_wave) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                     (__attribute__((address_space(3))) void*)dst_wave, 16, 0, 0);
}

template <int WTN>   // columns per wave: 128 (wide) or 64 (narrow)
__global__ __launch_bounds__(BG_THREADS, 2) void bgemm_big_kernel(const ffk_bgemm_desc d) {
    typedef Mma<T> MM;
    constexpr int BM = 256, BN = 2 * WTN;
    constexpr int NI = WTN / 32;                             // accumulator tiles along n per wave
    constexpr int ROWS = BM + BN;
    constexpr int NLD = ROWS * 4 / BG_THREADS;               // 16-byte loads per thread per chunk (4 or 3)
    constexpr int SLOT = ROWS * 64;                          // unpadded: rows of 64 bytes
    extern __shared__ __align__(16) unsigned char smem[];    // [BG_SLOTS][ROWS][64]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, half = lane >> 5;
    const int M = d.M, N = d.N, K = d.K;

    const unsigned tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const unsigned total = tiles_m * tiles_n * (unsigned)d.batch;
    const int kchunks = K / BG_BK;

    // Persistent workgroups.  Tile t of this workgroup: batched launches give every XCD a contiguous
    // eighth of the (batch, n-tile, m-tile) order (consecutive workgroup ids go to the eight XCDs in turn,
    // each with its own L2), so that all tiles of a batch run behind one L2; otherwise tiles are dealt
    // round-robin.  Returns false past the end.
    auto tile_at = [&](unsigned t, unsigned& item) {
        if (d.batch >= 8) {
            const unsigned per_xcd = (total + 7) >> 3, xcd = blockIdx.x & 7;
            const unsigned j = (blockIdx.x >> 3) + (gridDim.x >> 3) * t;
            item = xcd * per_xcd + j;
            return j < per_xcd && item < total;
        }
        item = blockIdx.x + gridDim.x * t;
        return item < total;
    };

    // ---- loader ----
    // Load i of a thread fills LDS position (row i*128 + wave*16 + lane/4, column lane%4) of a slot.
    // Rows 0..255 are A rows, the rest B rows.  Rows are unpadded, so to keep the fragment reads free of
    // bank conflicts position (row, c) holds global column  c ^ ((row >> 2) & 3)  of the chunk.
    // The chunk stream runs on across tiles: while the last chunks of one tile are multiplied and its
    // results stored, the first chunks of the next tile are already arriving.
    const T* src[NLD];
    unsigned f_t = 0;          // tile (of this workgroup) being fetched
    int f_kc = 0;              // next chunk of it
    unsigned g_fetch = 0;      // running chunk count -> ring slot
    auto fetch_setup = [&](unsigned item) {
        const long fm0 = (long)(item % tiles_m) * BM, fn0 = (long)((item / tiles_m) % tiles_n) * BN;
        const int fbz = (item / tiles_m) / tiles_n;
        const T* A = (const T*)d.a + (long)fbz * d.a_bs;
        const T* B = (const T*)d.b + (long)fbz * d.b_bs;
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int row = i * 128 + wave * 16 + (lane >> 2);
            const int g = (lane & 3) ^ ((row >> 2) & 3);
            if (i < BM / 128) {
                long m = fm0 + row;
                m = m < M ? m : M - 1;                       // clamped once; such rows are never stored
                src[i] = A + m * d.lda + g * 8;
            } else {
                long n = fn0 + row - BM;
                n = n < N ? n : N - 1;
                src[i] = B + n * d.ldb + g * 8;
            }
        }
    };
    auto fetch_next = [&]() {
        unsigned char* slot = smem + (g_fetch & (BG_SLOTS - 1)) * SLOT + wave * 1024;
#pragma unroll
        for (int i = 0; i < NLD; ++i) bg_load_lds(src[i] + f_kc * BG_BK, slot + i * 8192);
        ++g_fetch;
        if (++f_kc == kchunks) {                             // on to the next tile; past the last one the
            unsigned item;                                   // same chunks are re-read into free slots (harmless)
            f_kc = 0;
            if (tile_at(f_t + 1, item)) {
                ++f_t;
                fetch_setup(item);
            }
        }
    };
    // fragment addresses: A rows in natural order, B rows through tau; column (2 ks + half) un-swizzled
    const int ra = wm * 64 + l32, rb = BM + wn * WTN + bg_tau(l32);
    int fa_off[2], fb_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        fa_off[ks] = ra * 64 + (((2 * ks + half) ^ ((ra >> 2) & 3)) << 4);
        fb_off[ks] = rb * 64 + (((2 * ks + half) ^ ((rb >> 2) & 3)) << 4);
    }

    unsigned item;
    if (!tile_at(0, item)) return;                           // whole workgroup leaves together
    fetch_setup(item);
    fetch_next();
    fetch_next();
    fetch_next();
    unsigned g_use = 0;
    f32x16 acc[NI][2];   // [ni][mi]
    bf16x8 fa0[2], fb0[NI], fa1[2], fb1[NI];                 // fragments of K step 0 and of K step 1 of a chunk
    auto zero_acc = [&]() {
#pragma unroll
        for (int a = 0; a < NI; ++a)
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.0f;
    };
    auto read_frag = [&](const unsigned char* s, int ks, bf16x8 (&fa)[2], bf16x8 (&fb)[NI]) {
#pragma unroll
        for (int i = 0; i < 2; ++i) fa[i] = *reinterpret_cast<const bf16x8*>(s + fa_off[ks] + i * 32 * 64);
#pragma unroll
        for (int i = 0; i < NI; ++i) fb[i] = *reinterpret_cast<const bf16x8*>(s + fb_off[ks] + i * 32 * 64);
    };
    auto mma_half = [&](const bf16x8 (&fa)[2], const bf16x8 (&fb)[NI], int h) {
#pragma unroll
        for (int ni = h * (NI / 2); ni < (h + 1) * (NI / 2); ++ni)
#pragma unroll
            for (int mi = 0; mi < 2; ++mi) MM::mma(acc[ni][mi], fb[ni], fa[mi]);
    };
    auto epilogue = [&](long m0, long n0, int bz) {
    // ---- epilogue from registers: lane = row, registers = 16 consecutive columns ----
    T* out = (T*)d.out + (long)bz * d.o_bs;
    const T* resid = d.resid ? (const T*)d.resid + (long)bz * d.o_bs : nullptr;
    const T* bias = (const T*)d.bias;
    int8_t* xtail = d.xtail ? (int8_t*)d.xtail + (long)bz * d.o_bs : nullptr;   // extended residual stream (needs resid)
    const bool plain = !bias && !resid && d.act == FFK_ACT_NONE;
    const bool bias_resid = bias && resid && d.act == FFK_ACT_NONE && !xtail;
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
        const long m = m0 + wm * 64 + mi * 32 + l32;
        const bool mok = m < M;
        const unsigned mc = (unsigned)(mok ? m : M - 1);
        unsigned hi = 0, lo = mc;
        if ((unsigned)d.inner < (unsigned)M) {
            hi = mc / (unsigned)d.inner;
            lo = mc - hi * (unsigned)d.inner;
        }
        const long roff = (long)hi * d.s_o + (long)lo * d.s_i;
        float mul = d.scale;
        if (d.rowdiv) mul /= d.rowdiv[(long)bz * M + mc] + d.div_eps;
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
            const long n = n0 + wn * WTN + ni * 32 + 16 * half;      // first of this lane's 16 columns
            const bool ok0 = mok && n + 8 <= N, ok1 = mok && n + 16 <= N;
            const long nc = n + 16 <= N ? n : (N >= 16 ? N - 16 : 0);   // clamped for loads
            const long o = roff + (n >> 5) * d.s_h + (n & 31);
            const long oc = roff + (nc >> 5) * d.s_h + (nc & 31);
            // The three uniform switches (bias, residual, activation) are resolved once per block of 16 columns:
            // the two common combinations get straight-line code, anything else the general loop.
            T y[16];
            if (plain) {                                     // contraction: scale only
#pragma unroll
                for (int v = 0; v < 16; ++v) y[v] = (T)(acc[ni][mi][v] * mul);
            } else if (bias_resid) {                         // projection back onto the residual stream
                u32x4 bv[2], rv[2];
                bv[0] = *reinterpret_cast<const u32x4*>(bias + nc);
                bv[1] = *reinterpret_cast<const u32x4*>(bias + nc + 8);
                rv[0] = *reinterpret_cast<const u32x4*>(resid + oc);
                rv[1] = *reinterpret_cast<const u32x4*>(resid + oc + 8);
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const float x = (acc[ni][mi][v] + (float)reinterpret_cast<const T*>(&bv[v >> 3])[v & 7]) * mul;
                    y[v] = (T)((float)(T)x + (float)reinterpret_cast<const T*>(&rv[v >> 3])[v & 7]);
                }
            } else {
                u32x4 bv[2], rv[2];
                if (bias) {
                    bv[0] = *reinterpret_cast<const u32x4*>(bias + nc);
                    bv[1] = *reinterpret_cast<const u32x4*>(bias + nc + 8);
                }
                if (resid) {
                    rv[0] = *reinterpret_cast<const u32x4*>(resid + oc);
                    rv[1] = *reinterpret_cast<const u32x4*>(resid + oc + 8);
                }
                float upd[16];
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    float x = acc[ni][mi][v];
                    if (bias) x += (float)reinterpret_cast<const T*>(&bv[v >> 3])[v & 7];
                    if (d.act == FFK_ACT_RELU) x = relu_f(x);
                    else if (d.act == FFK_ACT_SIGMOID) x = sigmoid_f(x);
                    x *= mul;
                    upd[v] = (float)(T)x;        // the update rounded to bf16, as every variant of this epilogue does
                    if (resid) x = (float)(T)x + (float)reinterpret_cast<const T*>(&rv[v >> 3])[v & 7];
                    y[v] = (T)x;
                }
                if (xtail) {       // the update is added to the 24-bit value instead (tails: 16 bytes at the element offset)
                    const u32x4 tv = *reinterpret_cast<const u32x4*>(xtail + oc);
                    u32x4 h0, h1, tn;
                    xs_update16(upd, rv[0], rv[1], tv, h0, h1, tn);
                    if (ok1) {     // all 16 columns or none (N % 16 == 0 is required with a tail)
                        *reinterpret_cast<u32x4*>(out + o) = h0;
                        *reinterpret_cast<u32x4*>(out + o + 8) = h1;
                        *reinterpret_cast<u32x4*>(xtail + o) = tn;
                    }
                    continue;
                }
            }
            if (ok0) *reinterpret_cast<u32x4*>(out + o) = *reinterpret_cast<const u32x4*>(&y[0]);
            if (ok1) *reinterpret_cast<u32x4*>(out + o + 8) = *reinterpret_cast<const u32x4*>(&y[8]);
        }
    }
    };
    bool relaxed = false;      // previous tile was full: its stores are counted exactly
    for (unsigned t = 0; tile_at(t, item); ++t) {
        const long m0 = (long)(item % tiles_m) * BM, n0 = (long)((item / tiles_m) % tiles_n) * BN;
        const int bz = (item / tiles_m) / tiles_n;
        zero_acc();
        // One step = one chunk: wait, barrier, then the second K step of the chunk before (fragments fa1 / fb1), the
        // request for the chunk three ahead, and the first K step of this chunk.
        // Before the barrier: this wave's loads of the chunk have landed, and its fragment reads of the chunk before
        // have returned (lgkmcnt), so behind the barrier that slot is free for every wave's next request.
        // Loads and stores complete in the order of issue: the chunk has landed once at most the loads of the two
        // younger chunks are outstanding.  Right after a tile whose every store was issued (a full tile: no lane
        // predicate can have skipped one) those 4 * NI stores are known to be younger than the chunks awaited in the
        // first three steps and need not be waited for.
        auto wait_chunk = [&](bool after_full_tile) {
            if (after_full_tile) {
                if (NLD == 4) asm volatile("s_waitcnt vmcnt(24) lgkmcnt(0)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(14) lgkmcnt(0)" ::: "memory");
            } else {
                if (NLD == 4) asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)" ::: "memory");
            }
        };
        auto step = [&](bool first) {                        // known at every call site
            __builtin_amdgcn_s_barrier();
            const unsigned char* s = smem + (g_use & (BG_SLOTS - 1)) * SLOT;
            ++g_use;
            if (!first) {
                mma_half(fa1, fb1, 0);                       // second K step of the chunk before
                __builtin_amdgcn_sched_barrier(0);
            }
            read_frag(s, 0, fa0, fb0);
            fetch_next();
            __builtin_amdgcn_sched_barrier(0);
            if (!first) mma_half(fa1, fb1, 1);
            mma_half(fa0, fb0, 0);
            __builtin_amdgcn_sched_barrier(0);
            read_frag(s, 1, fa1, fb1);
            __builtin_amdgcn_sched_barrier(0);
            mma_half(fa0, fb0, 1);
            __builtin_amdgcn_sched_barrier(0);               // these MFMAs cover the reads the next wait asks for
        };
        wait_chunk(relaxed);
        step(true);
        wait_chunk(relaxed);
        step(false);
        wait_chunk(relaxed);
        step(false);
        for (int kc = 3; kc < kchunks; ++kc) {
            wait_chunk(false);
            step(false);
        }
        mma_half(fa1, fb1, 0);
        mma_half(fa1, fb1, 1);
        epilogue(m0, n0, bz);
        relaxed = m0 + BM <= M && n0 + BN <= N;
    }   // tiles
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");         // the re-reads past the end
}

template <int WTN>
int bg_launch(const ffk_bgemm_desc& d, hipStream_t st) {
    constexpr int BM = 256, BN = 2 * WTN;
    const size_t smem = (size_t)BG_SLOTS * (BM + BN) * 64;
    static FfkLdsReservation lds_reserved;
    {
        const int rc_lds = ffk_reserve_lds(lds_reserved, (const void*)bgemm_big_kernel<WTN>, smem, "ffk_bgemm_nt");
        if (rc_lds != FFK_OK) return rc_lds;
    }
    const long tiles = (long)ffk_cdiv(d.M, BM) * ffk_cdiv(d.N, BN) * d.batch;
    if (tiles >= (1L << 31) - 8) return ffk_fail(FFK_ERR_SHAPE, "ffk_bgemm_nt: %ld output tiles exceed the grid limit", tiles);
    const unsigned grid = (unsigned)(tiles < 256 ? 8 * ffk_cdiv(tiles, 8) : 256);   // persistent: one workgroup per CU
    bgemm_big_kernel<WTN><<<grid, BG_THREADS, smem, st>>>(d);
    return ffk_check_launch("ffk_bgemm_nt");
}

}  // namespace

// Launches the large-tile kernel if it can take this (already validated) descriptor and returns 1 with
// the launch status in *status; returns 0 if the caller has to use the small-tile kernel.
int ffk_bgemm_big_try(const ffk_bgemm_desc* d, hipStream_t st, int* status) {
    if (d->dtype != FFK_BF16 || d->out_f32 || d->K % BG_BK != 0 || d->K < 3 * BG_BK || d->s_d != 1) return 0;
    if (d->M < 256 || d->N < 64 || d->N % 16 != 0) return 0;
    if (d->xtail && (!d->resid || (reinterpret_cast<uintptr_t>(d->xtail) & 15) != 0)) return 0;
    auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    if (!al16(d->out) || (d->resid && !al16(d->resid)) || (d->bias && !al16(d->bias))) return 0;
    if (d->s_o % 8 || d->s_i % 8 || d->s_h % 8 || d->o_bs % 8) return 0;
    if (d->s_h != 32 && d->N % 32 != 0) return 0;            // 32-column blocks must be whole when they are strided
    // 256 x 256 tiles, unless they would leave CUs without a tile while 256 x 128 tiles would not (small batched launches)
    const long wide_tiles = (long)ffk_cdiv(d->M, 256) * ffk_cdiv(d->N, 256) * d->batch;
    const bool narrow = d->N <= 128 || (wide_tiles < 256 && d->N % 128 == 0);
    *status = narrow ? bg_launch<64>(*d, st) : bg_launch<128>(*d, st);
    return 1;
}
