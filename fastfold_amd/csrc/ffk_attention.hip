// Flash-style attention for head dimension 32 (see ffk_attention_fwd in include/ffk.h).
//
// One wavefront owns 32 queries of one (b2, head) and walks the keys 32 at a time.  Every
// operand is stored in HBM in exactly the order a wave consumes it (1024-element tiles, 16
// contiguous elements per lane); the eight waves of a workgroup share their operand tiles
// through a double-buffered LDS stage (see attention_kernel).
//
// The score tile is computed transposed, S^T = K . Q^T (rows = keys, columns = queries):
// a lane then holds 16 keys of ONE query, so the running max / sum are per-lane scalars
// (one cross-half shuffle per tile), and exp2(S^T - max) is already in the operand layout
// of the second MFMA  O^T += V^T . P^T  - no transpose of P.  The additive bias tile is
// stored as an MFMA operand (keys x queries) and added to S^T by one more MFMA against the
// identity: the matrix pipe has slack here (head dim 32 makes the kernel VALU / exp bound), the
// vector pipe has none.  Per-tile flags skip the key-mask add for tiles without masked keys and
// drop trailing fully-masked tiles; the running output is rescaled only when a row maximum moves.
#include "ffk_common.h"
#include <type_traits>

namespace {

constexpr int THREADS = 256;
constexpr float NEG_BIG = -3.0e38f;

template <typename T> struct Ops16 {   // the 16 elements one lane owns of a 1024-element tile
    static constexpr int NV = 16 / DT<T>::VEC;
    Vec16<T> v[NV];
    __device__ __forceinline__ void load(const T* p) {
#pragma unroll
        for (int i = 0; i < NV; ++i) v[i] = ld16(p + i * DT<T>::VEC);
    }
    // the same 16 elements from a tile kept in LDS vector-interleaved: vector i of lane l at (i * 64 + l)
    // * 16 bytes, so that the 64 lanes of one read touch 1 KB of consecutive addresses (the tile's own
    // order, 32 or 64 bytes from lane to lane, makes every 16-byte read a two- or four-way bank conflict)
    __device__ __forceinline__ void load_lds(const T* tile, int lane) {
#pragma unroll
        for (int i = 0; i < NV; ++i) v[i] = ld16(tile + (i * 64 + lane) * DT<T>::VEC);
    }
    __device__ __forceinline__ float f(int j) const { return DT<T>::to_f(v[j / DT<T>::VEC].e[j % DT<T>::VEC]); }
    // MFMA fragment number i (KLANE elements each)
    __device__ __forceinline__ typename Mma<T>::Frag frag(int i) const {
        return *reinterpret_cast<const typename Mma<T>::Frag*>(&v[i]);
    }
};

template <typename T> struct PFrag;
template <> struct PFrag<bf16_t> {
    static __device__ __forceinline__ bf16x8 make(const float* p) {
        bf16x8 r;
#pragma unroll
        for (int t = 0; t < 8; ++t) r[t] = (bf16_t)p[t];
        return r;
    }
    // acc + sum of the eight rounded probabilities (the values the PV product really uses), two
    // per instruction
    static __device__ __forceinline__ float add_sum(const bf16x8& f, float acc) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        const bf16x2 ones = {(bf16_t)1.0f, (bf16_t)1.0f};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const bf16x2 pr = {f[2 * t], f[2 * t + 1]};
            acc = __builtin_amdgcn_fdot2_f32_bf16(pr, ones, acc, false);
        }
        return acc;
    }
};
template <> struct PFrag<float> {
    static __device__ __forceinline__ f32x4 make(const float* p) {
        f32x4 r;
#pragma unroll
        for (int t = 0; t < 4; ++t) r[t] = p[t];
        return r;
    }
    static __device__ __forceinline__ float add_sum(const f32x4& f, float acc) {
        return acc + ((f[0] + f[1]) + (f[2] + f[3]));
    }
};

// One-hot fragments of the 32x32 identity in N-operand layout: lane (column q = l & 31, K-group
// kg = l >> 5) holds rows j = 16 * kg + i * KLANE + t; the entry is 1 where j == q.  Multiplying a
// bias tile stored in M-operand order by it adds the tile to the score accumulator on the matrix
// pipe, with no conversion or VALU work.
template <typename T>
__device__ __forceinline__ typename Mma<T>::Frag identity_frag(int i, int l32, int half) {
    typename Mma<T>::Frag f;
#pragma unroll
    for (int t = 0; t < Mma<T>::KLANE; ++t) f[t] = (T)((16 * half + i * Mma<T>::KLANE + t) == l32 ? 1.0f : 0.0f);
    return f;
}

// Workgroup = 8 wavefronts = 2 batch rows x 4 query tiles of one head.  Per 32-key step the
// workgroup needs the K and V tiles of its two batch rows and the bias tiles of its four query
// tiles: 8 operand tiles, each consumed by 4 (K, V) or 2 (bias) waves.  They are fetched from
// global memory once per workgroup (two 16-byte loads per thread), double-buffered in LDS, and read
// from there by the waves in exactly the lane order of the MFMA operands, which divides the
// traffic through the vector memory path by three compared with per-wave global loads.
constexpr int ATT_WAVES = 8;
constexpr int ATT_THREADS = 64 * ATT_WAVES;

template <typename T, bool HAS_BIAS>
__global__ __launch_bounds__(ATT_THREADS, sizeof(T) == 2 ? 4 : 2) void attention_kernel(
    T* __restrict__ out, const T* __restrict__ q_t, const T* __restrict__ k_t, const T* __restrict__ v_t,
    const T* __restrict__ bias_t, const float* __restrict__ keybias, const int* __restrict__ tileflags,
    const T* __restrict__ gate, int B2, int H, int Nq, int Nk, int flags) {
    typedef Mma<T> MM;
    typedef typename MM::Frag Frag;
    constexpr int NF = 16 / MM::KLANE;            // fragments per 16-element lane slice (bf16 2, fp32 4)
    constexpr int VEC = DT<T>::VEC;
    constexpr int NTILES = HAS_BIAS ? 8 : 4;      // operand tiles per key step: K0 K1 V0 V1 [B0 B1 B2 B3]
    constexpr int TILE_VECS = 1024 / VEC;         // 16-byte vectors per tile
    constexpr int NVL = (NTILES * TILE_VECS + ATT_THREADS - 1) / ATT_THREADS;   // vectors per thread per step
    extern __shared__ __align__(16) unsigned char att_smem[];
    constexpr int NSLOT = 3;                      // operand ring: the tile in use and two in flight behind it
    T* lds = reinterpret_cast<T*>(att_smem);      // [NSLOT][NTILES][1024] operand slots, then [ATT_THREADS][16] gate values

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: everything derived from it stays scalar
    const int l32 = lane & 31, half = lane >> 5;
    const int bsel = wave >> 2, qsel = wave & 3;
    const int QT = (Nq + 31) >> 5, KT = (Nk + 31) >> 5;
    // Workgroup -> work mapping.  The hardware hands consecutive workgroup ids to the eight XCDs in
    // turn, and each XCD has its own L2.  Logical work items are ordered (head, batch-row pair,
    // query group) and every XCD takes one contiguous eighth of that order, so that the query groups
    // that share a K / V pair and the batch rows that share a head's bias run behind the same L2.
    const int NQG = (QT + 3) >> 2, NZ = (B2 + 1) >> 1;
    const unsigned total = (unsigned)NQG * H * NZ, per_xcd = (total + 7) >> 3;
    const unsigned item = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (item >= total) return;                    // whole workgroup leaves together
    const int wg_q = item % NQG, wg_z = (item / NQG) % NZ;
    const int h = (item / NQG) / NZ;
    const int b2_raw = wg_z * 2 + bsel, qt_raw = wg_q * 4 + qsel;
    const bool live = b2_raw < B2 && qt_raw < QT;      // dead waves still help loading and keep the barriers
    const int b2 = b2_raw < B2 ? b2_raw : B2 - 1;
    const int qt = qt_raw < QT ? qt_raw : QT - 1;
    const long bh = (long)b2 * H + h;

    Ops16<T> qf;
    qf.load(q_t + ((bh * QT + qt) << 10) + lane * 16);
    const float* mp = keybias + (long)b2 * KT * 32 + 4 * half;
    const int* fl = tileflags + (long)b2 * KT;

    // cooperative operand fetch: vector slot v = tid + i * ATT_THREADS -> (tile, vector in tile).  The
    // 16-byte vectors go from global memory straight into LDS (no staging registers); the hardware places
    // the 64 vectors of a request at  base + 16 * lane,  while the source address is per lane: a request
    // gathers vector c of each lane's 16 elements (stride 16 * NV bytes), which leaves the tile in LDS
    // vector-interleaved (see Ops16::load_lds).
    static_assert(NVL * ATT_THREADS == NTILES * TILE_VECS, "every thread fetches the same number of vectors");
    const T* src[NVL];                            // wave-uniform: start of the wave's 64 vectors in key tile 0
#pragma unroll
    for (int i = 0; i < NVL; ++i) {
        const int v = wave * 64 + i * ATT_THREADS;
        const int tile = v / TILE_VECS, wv = v % TILE_VECS;
        const T* base;
        if (tile < 4) {
            int bb = wg_z * 2 + (tile & 1);
            bb = bb < B2 ? bb : B2 - 1;
            base = (tile < 2 ? k_t : v_t) + ((((long)bb * H + h) * KT) << 10);
        } else {
            int qq = wg_q * 4 + (tile - 4);
            qq = qq < QT ? qq : QT - 1;
            // FFK_ATT_BIAS_PADDED: one unused tile after the KT tiles of each query-tile row
            base = bias_t + ((((long)h * QT + qq) * (KT + ((flags >> 1) & 1))) << 10);
        }
        // the wave's 64 vectors of this request: vector number wv / 64 of every lane's 16 elements
        src[i] = base + (wv / 64) * VEC;
    }

    // gate values of this lane's 16 outputs, fetched now so that their latency is hidden by the loop
    const int q = qt * 32 + l32;
    const int qc = q < Nq ? q : Nq - 1;
    const long rowo = ((long)b2 * Nq + qc) * (H * 32) + h * 32 + 4 * half;
    // They wait in LDS (each lane's own 16 values), not in registers.
    T* gate_lds = lds + NSLOT * NTILES * 1024 + tid * 16;
    if (gate) {
        T gv[4][4];
        if (flags & FFK_ATT_GATE_TILED) {
            // accumulator-order tile: this lane's 16 values are contiguous
            const T* gp = gate + ((bh * QT + qt) << 10) + lane * 16;
            if (sizeof(T) == 2) {
                *reinterpret_cast<u32x4*>(&gv[0][0]) = *reinterpret_cast<const u32x4*>(gp);
                *reinterpret_cast<u32x4*>(&gv[2][0]) = *reinterpret_cast<const u32x4*>(gp + 8);
            } else {
#pragma unroll
                for (int g = 0; g < 4; ++g) *reinterpret_cast<u32x4*>(&gv[g][0]) = *reinterpret_cast<const u32x4*>(gp + 4 * g);
            }
        } else {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                if (sizeof(T) == 2) {
                    *reinterpret_cast<u32x2*>(&gv[g][0]) = *reinterpret_cast<const u32x2*>(gate + rowo + 8 * g);
                } else {
                    *reinterpret_cast<u32x4*>(&gv[g][0]) = *reinterpret_cast<const u32x4*>(gate + rowo + 8 * g);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 16 / VEC; ++i)
            *reinterpret_cast<u32x4*>(gate_lds + i * VEC) = *reinterpret_cast<const u32x4*>(&gv[0][0] + i * VEC);
    }

    // trailing key tiles that are completely masked in both batch rows contribute exactly zero
    int kt_end = KT;
    {
        const int* f0 = tileflags + (long)(wg_z * 2 < B2 ? wg_z * 2 : B2 - 1) * KT;
        const int* f1 = tileflags + (long)(wg_z * 2 + 1 < B2 ? wg_z * 2 + 1 : B2 - 1) * KT;
        while (kt_end > 1 && f0[kt_end - 1] == 2 && f1[kt_end - 1] == 2) --kt_end;
    }

    Frag ident[NF];
    if (HAS_BIAS) {
#pragma unroll
        for (int i = 0; i < NF; ++i) ident[i] = identity_frag<T>(i, l32, half);
    }

    // Online softmax with a lazily updated reference.  Instead of subtracting the running row maximum
    // from every score on the vector pipe, the negated reference  -m_ref[q]  is the C operand of the
    // first MFMA of each tile, so the accumulator already holds  s - m_ref  and exp2 is applied to it
    // directly.  m_ref is only moved (and O / l rescaled) when the probabilities of a tile show that
    // a score lies more than REF_SLACK above it, which bounds  p = exp2(s - m_ref) <= 2^REF_SLACK
    // in everything that is accumulated;  the first tile always sets it.
    constexpr float REF_SLACK = 20.0f;
    constexpr float REF_LIMIT = 1048576.0f;       // 2^REF_SLACK
    constexpr float REF_FLOOR = -1.0e4f;          // keeps m_ref small when the first tile is fully masked
    f32x16 o_acc, negm;
#pragma unroll
    for (int v = 0; v < 16; ++v) o_acc[v] = negm[v] = 0.0f;
    float l_run = 0.0f;                           // partial row sum of this lane's 16 keys per tile
    bool first = true;

    // The loads are issued from an asm statement on purpose: the compiler orders every later LDS read
    // after all outstanding loads of this kind it knows of (a full s_waitcnt vmcnt(0) right behind
    // the issue), while here the slot being filled is never the slot being read.  The explicit wait
    // at the top of the loop is what orders them.
    const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)att_smem;
    const unsigned lane_off = lane * 16 * Ops16<T>::NV;   // byte offset of this lane's 16 elements; the base address is scalar
    auto fetch = [&](int kt, int slot) {
#pragma unroll
        for (int i = 0; i < NVL; ++i) {
            const T* gp = src[i] + ((long)kt << 10);
            const unsigned dst = lds_base + (slot * NTILES * TILE_VECS + wave * 64 + i * ATT_THREADS) * 16;
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(gp), "s"(dst)
                         : "memory", "m0");
#pragma clang diagnostic pop
        }
    };

    // Every load the compiler knows of (q fragments, gate) is made to complete here: a wait it would
    // otherwise place at the first use inside the loop would also wait for the operand loads issued
    // just before that use.
#pragma unroll
    for (int i = 0; i < Ops16<T>::NV; ++i) asm volatile("" : "+v"(*reinterpret_cast<u32x4*>(&qf.v[i])));
    // The walk over the key tiles.  CAREFUL = false is the common case: the first tile sets the reference and no
    // later tile looks at its probabilities - the row sum is tested once, after the walk (see below).
    auto walk = [&](auto careful_c) {
    constexpr bool CAREFUL = decltype(careful_c)::value;
    fetch(0, 0);
    fetch(kt_end > 1 ? 1 : 0, 1);
    int flag_nxt = fl[0];
    int slot = 0;                                 // ring slot of tile kt
    for (int kt = 0; kt < kt_end; ++kt) {
        // Tile kt was requested two steps ago: wait until only the newest request (tile kt + 1) of this
        // thread is still in flight, then the barrier publishes tile kt and retires the slot of tile kt - 1.
        if (NVL == 1) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
        else if (NVL == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        const int flag = __builtin_amdgcn_readfirstlane(flag_nxt);
        lds_barrier();
        const int nxt = kt + 1 < kt_end ? kt + 1 : kt;
        const int nxt2 = kt + 2 < kt_end ? kt + 2 : kt_end - 1;
        fetch(nxt2, slot == 0 ? 2 : slot - 1);    // (slot + 2) % 3: the slot tile kt - 1 was read from
        flag_nxt = fl[nxt];
        const T* buf = lds + slot * NTILES * 1024;
        slot = slot == 2 ? 0 : slot + 1;
        Ops16<T> vc;
        vc.load_lds(buf + (2 + bsel) * 1024, lane);

        // S^T - m_ref = K . Q^T + Bias^T . I + (-m_ref)   (rows: keys, columns: queries)
        f32x16 s;
        auto score_tile = [&]() {
            Ops16<T> kc, bc;
            kc.load_lds(buf + bsel * 1024, lane);
            if (HAS_BIAS) bc.load_lds(buf + (4 + qsel) * 1024, lane);
            s = negm;
            // FFK_ATT_HALF_K: elements 8 .. 15 of every lane's sixteen are zero padding in q and k (narrow heads): the
            // second half of the score product adds nothing and is skipped
#pragma unroll
            for (int i = 0; i < NF / 2; ++i) MM::mma(s, kc.frag(i), qf.frag(i));
            if (!(flags & FFK_ATT_HALF_K)) {
#pragma unroll
                for (int i = NF / 2; i < NF; ++i) MM::mma(s, kc.frag(i), qf.frag(i));
            }
            if (HAS_BIAS) {
#pragma unroll
                for (int i = 0; i < NF; ++i) MM::mma(s, bc.frag(i), ident[i]);
            }
            if (flag != 0) {         // some key of this tile is masked or padding: add the key bias
                f32x4 mk[4];
#pragma unroll
                for (int g = 0; g < 4; ++g) mk[g] = *reinterpret_cast<const f32x4*>(mp + kt * 32 + 8 * g);
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int e = 0; e < 4; ++e) s[4 * g + e] += mk[g][e];
            }
        };
        // P^T = exp2(S^T - m_ref) rounded to the operand type, and the sum of this lane's 16 rounded values
        Frag pf[NF];
        float tsum;
        auto prob_tile = [&]() {
            float p[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) p[v] = fast_exp2(s[v]);
            tsum = 0.0f;
#pragma unroll
            for (int i = 0; i < NF; ++i) {
                pf[i] = PFrag<T>::make(p + i * MM::KLANE);
                tsum = PFrag<T>::add_sum(pf[i], tsum);
            }
        };
        // No maximum is taken on the common path: probabilities are non-negative, so a partial row sum
        // within 2^REF_SLACK proves that no score of the tile is more than REF_SLACK above the reference.
        // Only when some lane's sum exceeds that (or on the first tile, which sets the reference) is
        // the tile recomputed from its LDS slot, the reference moved to the row maximum and O / l rescaled.
        score_tile();
        bool move_ref = first;
        if (!first) {
            prob_tile();
            if (CAREFUL) {
                move_ref = __builtin_amdgcn_ballot_w64(!(tsum <= REF_LIMIT)) != 0;
                if (move_ref) score_tile();
            }
        }
        if (move_ref) {
            float mt = fmaxf(s[0], s[1]);
#pragma unroll
            for (int v = 2; v < 16; ++v) mt = fmaxf(mt, s[v]);
            const float mfull = fmaxf(mt, lane_xor<32>(mt));
            const float delta = first ? fmaxf(mfull, REF_FLOOR) : fmaxf(mfull, 0.0f);
            const float alpha = first ? 1.0f : fast_exp2(-delta);   // nothing accumulated before the first tile
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                s[v] -= delta;
                negm[v] -= delta;
                o_acc[v] *= alpha;
            }
            l_run *= alpha;
            first = false;
            prob_tile();
        }
        l_run += tsum;
        // O^T += V^T . P^T   (rows: head dim, columns: queries)
#pragma unroll
        for (int i = 0; i < NF; ++i) MM::mma(o_acc, vc.frag(i), pf[i]);

    }
    // the requests past the last tile must have landed before the ring is reused or handed on
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };

    // Optimistic walk first.  Probabilities are non-negative, so a finite row sum within 2^OPT_SLACK proves that
    // no score of the row lay more than OPT_SLACK (log2 units) above the first tile's maximum: nothing overflowed,
    // and fp32 accumulation keeps its relative precision at any such scale.  Otherwise (steeply rising scores, a
    // first tile that is completely masked) the whole workgroup walks again with the reference moved tile by tile.
    walk(std::false_type());
    {
        constexpr float OPT_LIMIT = 1.8446744e19f;    // 2^64
        int* redo = reinterpret_cast<int*>(lds + NSLOT * NTILES * 1024 + ATT_THREADS * 16);
        if (tid == 0) *redo = 0;
        lds_barrier();
        const bool bad = __builtin_amdgcn_ballot_w64(!(l_run <= OPT_LIMIT)) != 0;
        if (bad && lane == 0) *redo = 1;
        lds_barrier();
        if (*redo != 0) {                              // workgroup-uniform
            lds_barrier();
#pragma unroll
            for (int v = 0; v < 16; ++v) o_acc[v] = negm[v] = 0.0f;
            l_run = 0.0f;
            first = true;
            walk(std::true_type());
        }
    }

    // rows whose keys are all masked have l == 0 and produce zeros
    const float l_tot = l_run + lane_xor<32>(l_run);
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    if (live && q < Nq) {
        T gv[4][4];
        if (gate) {
#pragma unroll
            for (int i = 0; i < 16 / VEC; ++i)
                *reinterpret_cast<u32x4*>(&gv[0][0] + i * VEC) = *reinterpret_cast<const u32x4*>(gate_lds + i * VEC);
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            T r4[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float x = o_acc[4 * g + e] * inv;
                if (gate) x *= DT<T>::to_f(gv[g][e]);
                r4[e] = DT<T>::from_f(x);
            }
            if (sizeof(T) == 2) {
                *reinterpret_cast<u32x2*>(out + rowo + 8 * g) = *reinterpret_cast<const u32x2*>(r4);
            } else {
                *reinterpret_cast<u32x4*>(out + rowo + 8 * g) = *reinterpret_cast<const u32x4*>(r4);
            }
        }
    }
}

// Head dimensions 64 and 128 (the widths the reference's attention core also accepts; no module of the Evoformer
// uses them): the head is cut into DP = D / 32 parts of 32 channels, each part an operand tile of its own
// (part-major: part p of every tensor lies p * part elements behind part 0), so a score tile is the sum of DP
// products and the output DP accumulator tiles.  One wave per (batch row, head, 32 queries), operands straight
// from global memory, the classic running-maximum walk: this instantiation serves the stand-alone operator, not
// the inference block, and is not tuned beyond that.
template <typename T, int DP, bool HAS_BIAS>
__global__ __launch_bounds__(256) void attention_wide_kernel(
    T* __restrict__ out, const T* __restrict__ q_t, const T* __restrict__ k_t, const T* __restrict__ v_t,
    const T* __restrict__ bias_t, const float* __restrict__ keybias, const int* __restrict__ tileflags,
    int B2, int H, int Nq, int Nk, long part_q, long part_k) {
    typedef Mma<T> MM;
    typedef typename MM::Frag Frag;
    constexpr int NF = 16 / MM::KLANE;
    constexpr float REF_FLOOR = -1.0e4f;          // rows whose every score lies below are all-masked: they give zeros
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int QT = (Nq + 31) >> 5, KT = (Nk + 31) >> 5;
    const long item = (long)blockIdx.x * 4 + wave;
    if (item >= (long)B2 * H * QT) return;
    const int qt = (int)(item % QT);
    const long bh = item / QT;
    const int h = (int)(bh % H), b2 = (int)(bh / H);

    Ops16<T> qf[DP];
#pragma unroll
    for (int p = 0; p < DP; ++p) qf[p].load(q_t + p * part_q + ((bh * QT + qt) << 10) + lane * 16);
    const float* mp = keybias + (long)b2 * KT * 32 + 4 * half;
    const int* fl = tileflags + (long)b2 * KT;
    Frag ident[NF];
    if (HAS_BIAS) {
#pragma unroll
        for (int i = 0; i < NF; ++i) ident[i] = identity_frag<T>(i, l32, half);
    }
    f32x16 o_acc[DP];
#pragma unroll
    for (int p = 0; p < DP; ++p)
#pragma unroll
        for (int v = 0; v < 16; ++v) o_acc[p][v] = 0.0f;
    float m_run = REF_FLOOR, l_run = 0.0f;
    for (int kt = 0; kt < KT; ++kt) {
        if (fl[kt] == 2) continue;                 // every key masked or padding: contributes exactly zero
        f32x16 s;
#pragma unroll
        for (int v = 0; v < 16; ++v) s[v] = 0.0f;
#pragma unroll
        for (int p = 0; p < DP; ++p) {
            Ops16<T> kc;
            kc.load(k_t + p * part_k + ((bh * KT + kt) << 10) + lane * 16);
#pragma unroll
            for (int i = 0; i < NF; ++i) MM::mma(s, kc.frag(i), qf[p].frag(i));
        }
        if (HAS_BIAS) {
            Ops16<T> bc;
            bc.load(bias_t + ((((long)h * QT + qt) * KT + kt) << 10) + lane * 16);
#pragma unroll
            for (int i = 0; i < NF; ++i) MM::mma(s, bc.frag(i), ident[i]);
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const f32x4 mk = *reinterpret_cast<const f32x4*>(mp + kt * 32 + 8 * g);
#pragma unroll
            for (int e = 0; e < 4; ++e) s[4 * g + e] += mk[e];
        }
        float mt = fmaxf(s[0], s[1]);
#pragma unroll
        for (int v = 2; v < 16; ++v) mt = fmaxf(mt, s[v]);
        mt = fmaxf(mt, lane_xor<32>(mt));
        const float m_new = fmaxf(m_run, mt);
        const float alpha = fast_exp2(m_run - m_new);
        m_run = m_new;
        float pr[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) pr[v] = fast_exp2(s[v] - m_new);
        Frag pf[NF];
        float tsum = 0.0f;
#pragma unroll
        for (int i = 0; i < NF; ++i) {
            pf[i] = PFrag<T>::make(pr + i * MM::KLANE);
            tsum = PFrag<T>::add_sum(pf[i], tsum);
        }
        l_run = l_run * alpha + tsum;
#pragma unroll
        for (int p = 0; p < DP; ++p) {
            Ops16<T> vc;
            vc.load(v_t + p * part_k + ((bh * KT + kt) << 10) + lane * 16);
#pragma unroll
            for (int v = 0; v < 16; ++v) o_acc[p][v] *= alpha;
#pragma unroll
            for (int i = 0; i < NF; ++i) MM::mma(o_acc[p], vc.frag(i), pf[i]);
        }
    }
    const float l_tot = l_run + lane_xor<32>(l_run);
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    const int q = qt * 32 + l32;
    if (q < Nq) {
        T* o = out + ((long)b2 * Nq + q) * ((long)H * DP * 32) + (long)h * DP * 32 + 4 * half;
#pragma unroll
        for (int p = 0; p < DP; ++p)
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int e = 0; e < 4; ++e) o[p * 32 + 8 * g + e] = DT<T>::from_f(o_acc[p][4 * g + e] * inv);
    }
}

template <typename T, int DP>
int launch_attention_wide(void* out, const void* q, const void* k, const void* v, const void* bias, const float* kb,
                          const int* flags, long B2, long H, long Nq, long Nk, hipStream_t st) {
    const long QT = (Nq + 31) / 32, KT = (Nk + 31) / 32;
    const long grid = (B2 * H * QT + 3) / 4;
    FFK_REQUIRE(grid < (1L << 31), FFK_ERR_SHAPE, "ffk_attention_fwd: too many tiles for one launch");
    const long part_q = B2 * H * QT * 1024, part_k = B2 * H * KT * 1024;
    if (bias)
        attention_wide_kernel<T, DP, true><<<(unsigned)grid, 256, 0, st>>>((T*)out, (const T*)q, (const T*)k, (const T*)v,
                                                                         (const T*)bias, kb, flags, (int)B2, (int)H,
                                                                         (int)Nq, (int)Nk, part_q, part_k);
    else
        attention_wide_kernel<T, DP, false><<<(unsigned)grid, 256, 0, st>>>((T*)out, (const T*)q, (const T*)k, (const T*)v,
                                                                          nullptr, kb, flags, (int)B2, (int)H, (int)Nq,
                                                                          (int)Nk, part_q, part_k);
    return ffk_check_launch("ffk_attention_fwd");
}

// One thread block per batch row: writes the additive key bias and, per 32-key tile, a flag
// (0: all keys valid, 1: some masked / padding, 2: every key masked or padding).
template <typename T>
__global__ void key_bias_kernel(float* kb, int* flags, const T* mask, long N, long Npad, long sb, long sn) {
    const long b = blockIdx.x;
    for (long t0 = 0; t0 < Npad; t0 += blockDim.x) {
        const long k = t0 + threadIdx.x;           // blockDim.x is a multiple of 64, Npad of 32
        float v = 0.0f;
        if (k < Npad) {
            if (k >= N) v = NEG_BIG;
            else if (mask && DT<T>::to_f(mask[b * sb + k * sn]) == 0.0f) v = -1e9f * 1.4426950408889634f;
            kb[b * Npad + k] = v;
        }
        const unsigned long long bad = __builtin_amdgcn_ballot_w64(k < Npad && v != 0.0f);
        const int half = (threadIdx.x & 63) >> 5;
        const unsigned part = half ? (unsigned)(bad >> 32) : (unsigned)bad;
        if ((threadIdx.x & 31) == 0 && k < Npad) flags[b * (Npad >> 5) + (k >> 5)] = part == 0 ? 0 : (part == 0xffffffffu ? 2 : 1);
    }
}

template <typename T, bool HAS_BIAS>
int launch_attention_b(void* out, const void* q, const void* k, const void* v, const void* bias, const float* kb,
                       const int* flags, const void* gate, long B2, long H, long Nq, long Nk, int aflags, hipStream_t st) {
    const size_t smem = (3 * (size_t)(HAS_BIAS ? 8 : 4) * 1024 + ATT_THREADS * 16) * sizeof(T) + 16;   // operand ring + gate + redo flag
    static FfkLdsReservation lds_reserved;
    {
        const int rc_lds = ffk_reserve_lds(lds_reserved, (const void*)attention_kernel<T, HAS_BIAS>, smem, "ffk_attention_fwd");
        if (rc_lds != FFK_OK) return rc_lds;
    }
    const long items = (long)ffk_cdiv((Nq + 31) / 32, 4) * H * ffk_cdiv(B2, 2);
    FFK_REQUIRE(items < (1L << 31) - 8, FFK_ERR_SHAPE, "ffk_attention_fwd: %ld workgroups exceed the grid limit", items);
    dim3 grid((unsigned)(8 * ffk_cdiv(items, 8)));
    attention_kernel<T, HAS_BIAS><<<grid, ATT_THREADS, smem, st>>>((T*)out, (const T*)q, (const T*)k, (const T*)v,
                                                                  (const T*)bias, kb, flags, (const T*)gate, (int)B2,
                                                                  (int)H, (int)Nq, (int)Nk, aflags);
    return ffk_check_launch("ffk_attention_fwd");
}

template <typename T>
int launch_attention(void* out, const void* q, const void* k, const void* v, const void* bias, const float* kb,
                     const int* flags, const void* gate, long B2, long H, long Nq, long Nk, int aflags, hipStream_t st) {
    return bias ? launch_attention_b<T, true>(out, q, k, v, bias, kb, flags, gate, B2, H, Nq, Nk, aflags, st)
                : launch_attention_b<T, false>(out, q, k, v, nullptr, kb, flags, gate, B2, H, Nq, Nk, aflags, st);
}

}  // namespace

extern "C" int ffk_attention_fwd(void* out, const void* q_t, const void* k_t, const void* v_t, const void* bias_t,
                                 const float* keybias, const int32_t* tileflags, const void* gate, int64_t B2, int64_t H, int64_t Nq,
                                 int64_t Nk, int64_t D, int flags, int dtype, void* stream) {
    FFK_REQUIRE(out && q_t && k_t && v_t && keybias && tileflags, FFK_ERR_NULL, "ffk_attention_fwd: null pointer");
    FFK_REQUIRE(B2 > 0 && B2 < 131072 && H > 0 && H < 65536 && Nq > 0 && Nk > 0 && Nq < (1 << 24) && Nk < (1 << 24),
                FFK_ERR_SHAPE, "ffk_attention_fwd: bad shape B2=%ld H=%ld Nq=%ld Nk=%ld", (long)B2, (long)H, (long)Nq,
                (long)Nk);
    FFK_REQUIRE(ffk_aligned16(out) && ffk_aligned16(q_t) && ffk_aligned16(k_t) && ffk_aligned16(v_t) &&
                    ffk_aligned16(keybias) && (!bias_t || ffk_aligned16(bias_t)) && (!gate || ffk_aligned16(gate)),
                FFK_ERR_ALIGN, "ffk_attention_fwd: buffers must be 16-byte aligned");
    FFK_REQUIRE(D == 32 || D == 64 || D == 128, FFK_ERR_SHAPE,
                "ffk_attention_fwd: head dimension %ld (32, 64 or 128; narrower heads arrive zero-padded to 32)", (long)D);
    hipStream_t st = (hipStream_t)stream;
    if (D != 32) {
        FFK_REQUIRE(!gate && !(flags & (FFK_ATT_BIAS_PADDED | FFK_ATT_HALF_K)), FFK_ERR_UNSUPPORTED,
                    "ffk_attention_fwd: the gate, padded bias rows and the narrow-head flag are built for head dimension 32 only");
        if (dtype == FFK_BF16)
            return D == 64 ? launch_attention_wide<bf16_t, 2>(out, q_t, k_t, v_t, bias_t, keybias, tileflags, B2, H, Nq, Nk, st)
                           : launch_attention_wide<bf16_t, 4>(out, q_t, k_t, v_t, bias_t, keybias, tileflags, B2, H, Nq, Nk, st);
        if (dtype == FFK_F32)
            return D == 64 ? launch_attention_wide<float, 2>(out, q_t, k_t, v_t, bias_t, keybias, tileflags, B2, H, Nq, Nk, st)
                           : launch_attention_wide<float, 4>(out, q_t, k_t, v_t, bias_t, keybias, tileflags, B2, H, Nq, Nk, st);
        return ffk_fail(FFK_ERR_DTYPE, "ffk_attention_fwd: unsupported dtype tag %d", dtype);
    }
    switch (dtype) {
        case FFK_BF16: return launch_attention<bf16_t>(out, q_t, k_t, v_t, bias_t, keybias, tileflags, gate, B2, H, Nq, Nk, flags, st);
        case FFK_F32: return launch_attention<float>(out, q_t, k_t, v_t, bias_t, keybias, tileflags, gate, B2, H, Nq, Nk, flags, st);
        default: return ffk_fail(FFK_ERR_DTYPE, "ffk_attention_fwd: unsupported dtype tag %d", dtype);
    }
}

extern "C" int ffk_key_bias(float* keybias, int32_t* tileflags, const void* mask, int64_t B, int64_t N,
                            int64_t mask_sb, int64_t mask_sn, int dtype, void* stream) {
    FFK_REQUIRE(keybias && tileflags, FFK_ERR_NULL, "ffk_key_bias: null pointer");
    FFK_REQUIRE(B > 0 && N > 0 && B < (1L << 31), FFK_ERR_SHAPE, "ffk_key_bias: bad shape B=%ld N=%ld", (long)B, (long)N);
    const long Npad = (N + 31) / 32 * 32;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((unsigned)B);
    switch (dtype) {
        case FFK_BF16: key_bias_kernel<bf16_t><<<grid, 256, 0, st>>>(keybias, tileflags, (const bf16_t*)mask, N, Npad, mask_sb, mask_sn); break;
        case FFK_F32: key_bias_kernel<float><<<grid, 256, 0, st>>>(keybias, tileflags, (const float*)mask, N, Npad, mask_sb, mask_sn); break;
        case FFK_F16: key_bias_kernel<f16_t><<<grid, 256, 0, st>>>(keybias, tileflags, (const f16_t*)mask, N, Npad, mask_sb, mask_sn); break;
        default: return ffk_fail(FFK_ERR_DTYPE, "ffk_key_bias: unsupported dtype tag %d", dtype);
    }
    return ffk_check_launch("ffk_key_bias");
}
