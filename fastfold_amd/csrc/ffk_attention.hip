// Flash-style attention for head dimension 32 (see ffk_attention_fwd in include/ffk.h).
//
// One wavefront owns 32 queries of one (b2, head) and walks the keys 32 at a time; the
// four waves of a workgroup take consecutive query tiles of the same (b2, head), so their
// K / V tile reads hit the same lines.  There is no LDS and no barrier: every operand is
// stored in HBM in exactly the order a wave consumes it (1024-element tiles, 16 contiguous
// elements per lane).
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
};
template <> struct PFrag<float> {
    static __device__ __forceinline__ f32x4 make(const float* p) {
        f32x4 r;
#pragma unroll
        for (int t = 0; t < 4; ++t) r[t] = p[t];
        return r;
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

template <typename T, bool HAS_BIAS>
__global__ __launch_bounds__(THREADS, sizeof(T) == 2 ? 3 : 2) void attention_kernel(T* __restrict__ out, const T* __restrict__ q_t,
                                                              const T* __restrict__ k_t, const T* __restrict__ v_t,
                                                              const T* __restrict__ bias_t,
                                                              const float* __restrict__ keybias,
                                                              const int* __restrict__ tileflags,
                                                              const T* __restrict__ gate, int H, int Nq, int Nk) {
    typedef Mma<T> MM;
    typedef typename MM::Frag Frag;
    constexpr int NF = 16 / MM::KLANE;            // fragments per 16-element lane slice (bf16 2, fp32 4)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int QT = (Nq + 31) >> 5, KT = (Nk + 31) >> 5;
    const int qt = blockIdx.x * 4 + wave;
    if (qt >= QT) return;
    const int h = blockIdx.y, b2 = blockIdx.z;
    const long bh = (long)b2 * H + h;

    Ops16<T> qf;
    qf.load(q_t + ((bh * QT + qt) << 10) + lane * 16);
    const T* kp = k_t + ((bh * KT) << 10) + lane * 16;
    const T* vp = v_t + ((bh * KT) << 10) + lane * 16;
    const T* bp = HAS_BIAS ? bias_t + ((((long)h * QT + qt) * KT) << 10) + lane * 16 : nullptr;
    const float* mp = keybias + (long)b2 * KT * 32 + 4 * half;
    const int* fl = tileflags + (long)b2 * KT;

    // gate values of this lane's 16 outputs, fetched now so that their latency is hidden by the loop
    const int q = qt * 32 + l32;
    const int qc = q < Nq ? q : Nq - 1;
    const long rowo = ((long)b2 * Nq + qc) * (H * 32) + h * 32 + 4 * half;
    T gv[4][4];
    if (gate) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            if (sizeof(T) == 2) {
                *reinterpret_cast<u32x2*>(&gv[g][0]) = *reinterpret_cast<const u32x2*>(gate + rowo + 8 * g);
            } else {
                *reinterpret_cast<u32x4*>(&gv[g][0]) = *reinterpret_cast<const u32x4*>(gate + rowo + 8 * g);
            }
        }
    }

    // trailing key tiles that are completely masked (sequence padding) contribute exactly zero
    int kt_end = KT;
    while (kt_end > 1 && fl[kt_end - 1] == 2) --kt_end;

    Frag ident[NF];
    if (HAS_BIAS) {
#pragma unroll
        for (int i = 0; i < NF; ++i) ident[i] = identity_frag<T>(i, l32, half);
    }

    // Online softmax with a lazily updated reference.  Instead of subtracting the running row maximum
    // from every score on the vector pipe, the negated reference  -m_ref[q]  is the C operand of the
    // first MFMA of each tile, so the accumulator already holds  s - m_ref  and exp2 is applied to it
    // directly.  m_ref is only moved (and O / l rescaled) when a tile contains a score more than
    // REF_SLACK above it, which bounds  p = exp2(s - m_ref) <= 2^REF_SLACK;  the first tile always
    // sets it.  The row sum l is accumulated on the matrix pipe as well (ones . P^T).
    constexpr float REF_SLACK = 20.0f;
    constexpr float REF_FLOOR = -1.0e4f;          // keeps m_ref small when the first tile is fully masked
    f32x16 o_acc, l_acc, negm;
#pragma unroll
    for (int v = 0; v < 16; ++v) o_acc[v] = l_acc[v] = negm[v] = 0.0f;
    bool first = true;
    Frag ones;
#pragma unroll
    for (int t = 0; t < MM::KLANE; ++t) ones[t] = (T)1.0f;

    auto load_tile = [&](int kt, Ops16<T>& kk, Ops16<T>& vv, Ops16<T>& bb) {
        kk.load(kp + ((long)kt << 10));
        vv.load(vp + ((long)kt << 10));
        if (HAS_BIAS) bb.load(bp + ((long)kt << 10));
    };

    auto process = [&](int kt, const Ops16<T>& kc, const Ops16<T>& vc, const Ops16<T>& bc) {
        // S^T - m_ref = K . Q^T + Bias^T . I + (-m_ref)   (rows: keys, columns: queries)
        f32x16 s = negm;
#pragma unroll
        for (int i = 0; i < NF; ++i) MM::mma(s, kc.frag(i), qf.frag(i));
        if (HAS_BIAS) {
#pragma unroll
            for (int i = 0; i < NF; ++i) MM::mma(s, bc.frag(i), ident[i]);
        }
        if (fl[kt] != 0) {           // some key of this tile is masked or padding: add the key bias
            f32x4 mk[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) mk[g] = *reinterpret_cast<const f32x4*>(mp + kt * 32 + 8 * g);
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int e = 0; e < 4; ++e) s[4 * g + e] += mk[g][e];
        }
        float mt = fmaxf(s[0], s[1]);
#pragma unroll
        for (int v = 2; v < 16; ++v) mt = fmaxf(mt, s[v]);
        if (first || __builtin_amdgcn_ballot_w64(mt > REF_SLACK) != 0) {
            // move the reference of every row of this wave to its running maximum
            const float mfull = fmaxf(mt, __shfl_xor(mt, 32, 64));
            const float delta = first ? fmaxf(mfull, REF_FLOOR) : fmaxf(mfull, 0.0f);
            const float alpha = first ? 1.0f : fast_exp2(-delta);   // nothing accumulated before the first tile
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                s[v] -= delta;
                negm[v] -= delta;
                o_acc[v] *= alpha;
            }
            l_acc[0] *= alpha;
            first = false;
        }
        float p[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) p[v] = fast_exp2(s[v]);
        // O^T += V^T . P^T  and  l += 1 . P^T   (rows: head dim, columns: queries)
#pragma unroll
        for (int i = 0; i < NF; ++i) {
            const Frag pf = PFrag<T>::make(p + i * MM::KLANE);
            MM::mma(o_acc, vc.frag(i), pf);
            MM::mma(l_acc, ones, pf);
        }
    };

    // Software pipeline over two register sets used alternately (no copies).  Every prefetch is
    // unconditional (the tile index is clamped instead), which keeps the loop free of branches
    // around loads so the compiler can wait for exactly the tile it needs.
    Ops16<T> ka, va, ba, kb, vb, bb;
    const int last = kt_end - 1;
    const int n2 = kt_end & ~1;
    load_tile(0, ka, va, ba);
    for (int kt = 0; kt < n2; kt += 2) {
        load_tile(kt + 1, kb, vb, bb);
        process(kt, ka, va, ba);
        load_tile(kt + 2 < last ? kt + 2 : last, ka, va, ba);
        process(kt + 1, kb, vb, bb);
    }
    if (kt_end & 1) process(last, ka, va, ba);

    // every row of l_acc holds the full row sum (the MFMA already summed both lane halves); rows whose
    // keys are all masked have l == 0 and produce zeros
    const float l_tot = l_acc[0];
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    if (q < Nq) {
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

template <typename T>
int launch_attention(void* out, const void* q, const void* k, const void* v, const void* bias, const float* kb,
                     const int* flags, const void* gate, long B2, long H, long Nq, long Nk, hipStream_t st) {
    dim3 grid(ffk_cdiv((Nq + 31) / 32, 4), (unsigned)H, (unsigned)B2);
    if (bias)
        attention_kernel<T, true><<<grid, THREADS, 0, st>>>((T*)out, (const T*)q, (const T*)k, (const T*)v,
                                                          (const T*)bias, kb, flags, (const T*)gate, (int)H, (int)Nq, (int)Nk);
    else
        attention_kernel<T, false><<<grid, THREADS, 0, st>>>((T*)out, (const T*)q, (const T*)k, (const T*)v, nullptr,
                                                           kb, flags, (const T*)gate, (int)H, (int)Nq, (int)Nk);
    return ffk_check_launch("ffk_attention_fwd");
}

}  // namespace

extern "C" int ffk_attention_fwd(void* out, const void* q_t, const void* k_t, const void* v_t, const void* bias_t,
                                 const float* keybias, const int32_t* tileflags, const void* gate, int64_t B2, int64_t H, int64_t Nq,
                                 int64_t Nk, int dtype, void* stream) {
    FFK_REQUIRE(out && q_t && k_t && v_t && keybias && tileflags, FFK_ERR_NULL, "ffk_attention_fwd: null pointer");
    FFK_REQUIRE(B2 > 0 && B2 < 65536 && H > 0 && H < 65536 && Nq > 0 && Nk > 0 && Nq < (1 << 24) && Nk < (1 << 24),
                FFK_ERR_SHAPE, "ffk_attention_fwd: bad shape B2=%ld H=%ld Nq=%ld Nk=%ld", (long)B2, (long)H, (long)Nq,
                (long)Nk);
    FFK_REQUIRE(ffk_aligned16(out) && ffk_aligned16(q_t) && ffk_aligned16(k_t) && ffk_aligned16(v_t) &&
                    ffk_aligned16(keybias) && (!bias_t || ffk_aligned16(bias_t)) && (!gate || ffk_aligned16(gate)),
                FFK_ERR_ALIGN, "ffk_attention_fwd: buffers must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case FFK_BF16: return launch_attention<bf16_t>(out, q_t, k_t, v_t, bias_t, keybias, tileflags, gate, B2, H, Nq, Nk, st);
        case FFK_F32: return launch_attention<float>(out, q_t, k_t, v_t, bias_t, keybias, tileflags, gate, B2, H, Nq, Nk, st);
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
