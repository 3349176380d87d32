// Backward of the attention core for head dimensions 32, 64 and 128 (see ffk_attention_bwd in include/ffk.h).
// A head wider than 32 is cut into DP = D / 32 parts of 32 channels, each with operand tiles of its own (part-major:
// part p of a tensor lies p * part elements behind part 0): scores and dP are sums over the parts, dq / dk / dv have one
// accumulator tile per part.
//
// Like the forward kernel it never forms the [B2, H, Nq, Nk] logits in memory: both kernels recompute the
// 32 x 32 score tiles from q and k on the matrix pipe.  With  s = q.k / sqrt(d) + bias  (masked keys very
// negative),  P = softmax_k(s),  o = P v  and the incoming gradient  do:
//     D[q]  = sum_d do[q, d] o[q, d]
//     dP    = do . v^T                 dS = P (dP - D)         (gradient w.r.t. the logits s)
//     dq    = dS . k / sqrt(d)         dk = dS^T . q / sqrt(d)
//     dv    = P^T . do                 dbias[h, q, k] = sum_b2 dS
//   attention_bwd_dq_kernel   one wave per (b2, head, 32 queries): a first walk over the key tiles finds the row
//                             maximum and sum (log2 domain, as the forward kernel) and D; they are written out for
//                             the second kernel.  The second walk accumulates dq^T = k^T . dS^T, the score tile
//                             transposed (keys along the MFMA rows) exactly as in the forward kernel, so that dS^T
//                             is the N operand of that product as it stands.
//   attention_bwd_dkv_kernel  one wave per (b2, head, 32 keys): walks the query tiles with the score tile the other
//                             way round (queries along the MFMA rows, one key per lane), so that P and dS are the N
//                             operands of  dv^T = do^T . P  and  dk^T = q^T . dS.
//   attention_bwd_dbias_kernel  one wave per (head, query tile, key tile, slice of the batch rows): recomputes dS of
//                             its tile for every batch row of the slice, sums in registers and adds the result to
//                             dbias with one fp32 atomic per element (the slices are what fills the chip when
//                             H * QT * KT alone is a few hundred tiles).
// Both take the pair bias from the same operand tiles as the forward kernel: added to the scores by a product with
// an identity operand, here with the roles of the two operands exchanged (rows = queries).
// Every operand arrives in the tile order its role needs (the wrapper re-tiles q, k, v, do with the same helpers
// as the forward pass); waves load their tiles straight from global memory - this pair of kernels serves the
// autograd path of the stand-alone operator, not the inference block, and is not tuned beyond that.
#include "ffk_common.h"

namespace {

constexpr float REF_FLOOR = -1.0e4f;          // as in the forward kernel: rows whose every score lies below are all-masked
constexpr float NO_ROW = 3.0e38f;             // log-sum-exp of a row without a valid key: exp2(s - NO_ROW) = 0

template <typename T> struct Tile16 {         // the 16 elements one lane owns of a 1024-element tile
    static constexpr int NV = 16 / DT<T>::VEC;
    Vec16<T> v[NV];
    __device__ __forceinline__ void load(const T* p) {
#pragma unroll
        for (int i = 0; i < NV; ++i) v[i] = ld16(p + i * DT<T>::VEC);
    }
    __device__ __forceinline__ float f(int j) const { return DT<T>::to_f(v[j / DT<T>::VEC].e[j % DT<T>::VEC]); }
    __device__ __forceinline__ typename Mma<T>::Frag frag(int i) const {
        return *reinterpret_cast<const typename Mma<T>::Frag*>(
            reinterpret_cast<const unsigned char*>(&v[0]) + i * sizeof(typename Mma<T>::Frag));
    }
};

// fragments (N operand) of 16 fp32 values held in accumulator order, rounded to the operand type
template <typename T> struct NFrag;
template <> struct NFrag<bf16_t> {
    static __device__ __forceinline__ bf16x8 make(const float* p) {
        bf16x8 r;
#pragma unroll
        for (int t = 0; t < 8; ++t) r[t] = (bf16_t)p[t];
        return r;
    }
};
template <> struct NFrag<float> {
    static __device__ __forceinline__ f32x4 make(const float* p) {
        f32x4 r;
#pragma unroll
        for (int t = 0; t < 4; ++t) r[t] = p[t];
        return r;
    }
};

template <typename T>
__device__ __forceinline__ typename Mma<T>::Frag identity_frag(int i, int l32, int half) {
    typename Mma<T>::Frag f;
#pragma unroll
    for (int t = 0; t < Mma<T>::KLANE; ++t) f[t] = (T)((16 * half + i * Mma<T>::KLANE + t) == l32 ? 1.0f : 0.0f);
    return f;
}

// Workgroup -> logical block.  The hardware hands consecutive workgroup ids to the eight XCDs in turn, each with its own
// L2; the launches round their grids up to a multiple of eight and every XCD takes a contiguous eighth of the logical
// order, so that the waves that walk the same k / v (or q / do) tiles run behind one L2.
__device__ __forceinline__ long bwd_logical_block() {
    const unsigned per_xcd = gridDim.x >> 3;
    return (long)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
}

// ------------------------------------------------------------------------------ dq ----
template <typename T, int DP, bool HAS_BIAS>
__global__ __launch_bounds__(256) void attention_bwd_dq_kernel(
    T* __restrict__ dq, float* __restrict__ lse, float* __restrict__ dsum, const T* __restrict__ q_qk,
    const T* __restrict__ k_qk, const T* __restrict__ k_acc, const T* __restrict__ v_qk, const T* __restrict__ bias_t,
    const float* __restrict__ keybias, const T* __restrict__ do_qk, const T* __restrict__ o_qk, int B2, int H, int Nq,
    int Nk, float dq_scale, long part_q, long part_k) {
    typedef Mma<T> MM;
    typedef typename MM::Frag Frag;
    constexpr int NF = 16 / MM::KLANE;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int QT = (Nq + 31) >> 5, KT = (Nk + 31) >> 5;
    const long item = bwd_logical_block() * 4 + wave;
    if (item >= (long)B2 * H * QT) return;
    const int qt = (int)(item % QT);
    const long bh = item / QT;
    const int h = (int)(bh % H), b2 = (int)(bh / H);

    Tile16<T> qf[DP], dof[DP];
    float dpart = 0.0f;
#pragma unroll
    for (int p = 0; p < DP; ++p) {
        Tile16<T> of;
        qf[p].load(q_qk + p * part_q + ((bh * QT + qt) << 10) + lane * 16);
        dof[p].load(do_qk + p * part_q + ((bh * QT + qt) << 10) + lane * 16);
        of.load(o_qk + p * part_q + ((bh * QT + qt) << 10) + lane * 16);
#pragma unroll
        for (int j = 0; j < 16; ++j) dpart += dof[p].f(j) * of.f(j);
    }
    const float D = dpart + lane_xor<32>(dpart);             // this lane's query: sum_d do o
    const float* mp = keybias + (long)b2 * KT * 32 + 4 * half;

    Frag ident[NF];
    if (HAS_BIAS) {
#pragma unroll
        for (int i = 0; i < NF; ++i) ident[i] = identity_frag<T>(i, l32, half);
    }
    // S^T tile kt (rows: keys, columns: queries), log2 domain, key bias included
    auto score = [&](int kt, f32x16& s) {
#pragma unroll
        for (int v = 0; v < 16; ++v) s[v] = 0.0f;
#pragma unroll
        for (int p = 0; p < DP; ++p) {
            Tile16<T> kc;
            kc.load(k_qk + p * part_k + ((bh * KT + kt) << 10) + lane * 16);
#pragma unroll
            for (int i = 0; i < NF; ++i) MM::mma(s, kc.frag(i), qf[p].frag(i));
        }
        if (HAS_BIAS) {
            Tile16<T> bc;
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
    };

    // first walk: row maximum and sum
    float m_run = REF_FLOOR, l_run = 0.0f;
    for (int kt = 0; kt < KT; ++kt) {
        f32x16 s;
        score(kt, s);
        float mt = fmaxf(s[0], s[1]);
#pragma unroll
        for (int v = 2; v < 16; ++v) mt = fmaxf(mt, s[v]);
        mt = fmaxf(mt, lane_xor<32>(mt));
        const float m_new = fmaxf(m_run, mt);
        float ts = 0.0f;
#pragma unroll
        for (int v = 0; v < 16; ++v) ts += fast_exp2(s[v] - m_new);
        l_run = l_run * fast_exp2(m_run - m_new) + ts;
        m_run = m_new;
    }
    const float l_tot = l_run + lane_xor<32>(l_run);
    const float L = l_tot > 0.0f ? m_run + __builtin_amdgcn_logf(l_tot) : NO_ROW;   // v_log_f32 is log2
    if (half == 0) {
        lse[(bh * QT + qt) * 32 + l32] = L;
        dsum[(bh * QT + qt) * 32 + l32] = D;
    }

    // second walk: dq^T += k^T . dS^T
    f32x16 acc[DP];
#pragma unroll
    for (int p = 0; p < DP; ++p)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[p][v] = 0.0f;
    for (int kt = 0; kt < KT; ++kt) {
        f32x16 s, dp;
        score(kt, s);
#pragma unroll
        for (int v = 0; v < 16; ++v) dp[v] = 0.0f;
#pragma unroll
        for (int p = 0; p < DP; ++p) {
            Tile16<T> vq;
            vq.load(v_qk + p * part_k + ((bh * KT + kt) << 10) + lane * 16);
#pragma unroll
            for (int i = 0; i < NF; ++i) MM::mma(dp, vq.frag(i), dof[p].frag(i));      // dP^T[key, q] = v[key] . do[q]
        }
        float ds[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) ds[v] = fast_exp2(s[v] - L) * (dp[v] - D);
        Frag dsf[NF];
#pragma unroll
        for (int i = 0; i < NF; ++i) dsf[i] = NFrag<T>::make(ds + i * MM::KLANE);
#pragma unroll
        for (int p = 0; p < DP; ++p) {
            Tile16<T> ka;
            ka.load(k_acc + p * part_k + ((bh * KT + kt) << 10) + lane * 16);
#pragma unroll
            for (int i = 0; i < NF; ++i) MM::mma(acc[p], ka.frag(i), dsf[i]);
        }
    }
    const int q = qt * 32 + l32;
    if (q < Nq) {
        T* o = dq + (bh * Nq + q) * (32 * DP) + 4 * half;
#pragma unroll
        for (int p = 0; p < DP; ++p)
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int e = 0; e < 4; ++e) o[32 * p + 8 * g + e] = DT<T>::from_f(acc[p][4 * g + e] * dq_scale);
    }
}

// ------------------------------------------------------------------------- dk, dv ----
template <typename T, int DP>
__global__ __launch_bounds__(256) void attention_bwd_dkv_kernel(
    T* __restrict__ dk, T* __restrict__ dv, const T* __restrict__ q_qk,
    const T* __restrict__ q_acc, const T* __restrict__ k_qk, const T* __restrict__ v_qk, const T* __restrict__ bias_t,
    const float* __restrict__ keybias, const T* __restrict__ do_qk, const T* __restrict__ do_acc,
    const float* __restrict__ lse, const float* __restrict__ dsum, int B2, int H, int Nq, int Nk, float dk_scale,
    long part_q, long part_k) {
    typedef Mma<T> MM;
    typedef typename MM::Frag Frag;
    constexpr int NF = 16 / MM::KLANE;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int QT = (Nq + 31) >> 5, KT = (Nk + 31) >> 5;
    const long item = bwd_logical_block() * 4 + wave;
    if (item >= (long)B2 * H * KT) return;
    const int kt = (int)(item % KT);
    const long bh = item / KT;
    const int h = (int)(bh % H), b2 = (int)(bh / H);

    Tile16<T> kf[DP], vf[DP];                      // this lane's key (column l32): k and v rows as N operands
#pragma unroll
    for (int p = 0; p < DP; ++p) {
        kf[p].load(k_qk + p * part_k + ((bh * KT + kt) << 10) + lane * 16);
        vf[p].load(v_qk + p * part_k + ((bh * KT + kt) << 10) + lane * 16);
    }
    const int key = kt * 32 + l32;
    const float kb = keybias[(long)b2 * KT * 32 + key];     // 0, masked (-1e9 log2e) or padding (hugely negative)
    Frag ident[NF];
    if (bias_t) {
#pragma unroll
        for (int i = 0; i < NF; ++i) ident[i] = identity_frag<T>(i, l32, half);
    }

    f32x16 acc_k[DP], acc_v[DP];
#pragma unroll
    for (int p = 0; p < DP; ++p)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc_k[p][v] = acc_v[p][v] = 0.0f;
    for (int qt = 0; qt < QT; ++qt) {
        f32x16 s, dp;
#pragma unroll
        for (int v = 0; v < 16; ++v) s[v] = dp[v] = 0.0f;
#pragma unroll
        for (int p = 0; p < DP; ++p) {
            Tile16<T> qc, doc;
            qc.load(q_qk + p * part_q + ((bh * QT + qt) << 10) + lane * 16);
            doc.load(do_qk + p * part_q + ((bh * QT + qt) << 10) + lane * 16);
#pragma unroll
            for (int i = 0; i < NF; ++i) MM::mma(s, qc.frag(i), kf[p].frag(i));       // S[q, key], log2 domain
#pragma unroll
            for (int i = 0; i < NF; ++i) MM::mma(dp, doc.frag(i), vf[p].frag(i));     // dP[q, key] = do[q] . v[key]
        }
        if (bias_t) {                                                           // S += I . bias (rows = queries)
            Tile16<T> bc;
            bc.load(bias_t + ((((long)h * QT + qt) * KT + kt) << 10) + lane * 16);
#pragma unroll
            for (int i = 0; i < NF; ++i) MM::mma(s, ident[i], bc.frag(i));
        }
        const float* lp = lse + (bh * QT + qt) * 32 + 4 * half;
        const float* dpz = dsum + (bh * QT + qt) * 32 + 4 * half;
        float p[16], ds[16];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const f32x4 L4 = *reinterpret_cast<const f32x4*>(lp + 8 * g);
            const f32x4 D4 = *reinterpret_cast<const f32x4*>(dpz + 8 * g);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int v = 4 * g + e;
                p[v] = fast_exp2(s[v] + kb - L4[e]);
                ds[v] = p[v] * (dp[v] - D4[e]);
            }
        }
        Frag pfr[NF], dsf[NF];
#pragma unroll
        for (int i = 0; i < NF; ++i) {
            pfr[i] = NFrag<T>::make(p + i * MM::KLANE);
            dsf[i] = NFrag<T>::make(ds + i * MM::KLANE);
        }
#pragma unroll
        for (int pp = 0; pp < DP; ++pp) {
            Tile16<T> qa, doa;
            qa.load(q_acc + pp * part_q + ((bh * QT + qt) << 10) + lane * 16);
            doa.load(do_acc + pp * part_q + ((bh * QT + qt) << 10) + lane * 16);
#pragma unroll
            for (int i = 0; i < NF; ++i) MM::mma(acc_v[pp], doa.frag(i), pfr[i]);   // dv^T += do^T . P
#pragma unroll
            for (int i = 0; i < NF; ++i) MM::mma(acc_k[pp], qa.frag(i), dsf[i]);    // dk^T += q^T . dS
        }
    }
    if (key < Nk) {
        T* ok = dk + (bh * Nk + key) * (32 * DP) + 4 * half;
        T* ov = dv + (bh * Nk + key) * (32 * DP) + 4 * half;
#pragma unroll
        for (int pp = 0; pp < DP; ++pp)
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    ok[32 * pp + 8 * g + e] = DT<T>::from_f(acc_k[pp][4 * g + e] * dk_scale);
                    ov[32 * pp + 8 * g + e] = DT<T>::from_f(acc_v[pp][4 * g + e]);
                }
    }
}

// ---------------------------------------------------------------------------- dbias ----
// dbias[h, q, key] += sum over the batch rows b2 = slice, slice + NS, ... of dS[b2, h, q, key].
template <typename T, int DP>
__global__ __launch_bounds__(256) void attention_bwd_dbias_kernel(
    float* __restrict__ dbias, const T* __restrict__ q_qk, const T* __restrict__ k_qk, const T* __restrict__ v_qk,
    const T* __restrict__ bias_t, const float* __restrict__ keybias, const T* __restrict__ do_qk,
    const float* __restrict__ lse, const float* __restrict__ dsum, int B2, int H, int Nq, int Nk, int NS,
    long part_q, long part_k) {
    typedef Mma<T> MM;
    typedef typename MM::Frag Frag;
    constexpr int NF = 16 / MM::KLANE;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int QT = (Nq + 31) >> 5, KT = (Nk + 31) >> 5;
    const long item = bwd_logical_block() * 4 + wave;          // key tile fastest: a block's waves share q and do
    if (item >= (long)NS * H * QT * KT) return;
    const int kt = (int)(item % KT);
    const int qt = (int)((item / KT) % QT);
    const int h = (int)((item / ((long)KT * QT)) % H);
    const int slice = (int)(item / ((long)KT * QT * H));
    const int key = kt * 32 + l32;

    Frag ident[NF];
#pragma unroll
    for (int i = 0; i < NF; ++i) ident[i] = identity_frag<T>(i, l32, half);
    Tile16<T> bc;
    bc.load(bias_t + ((((long)h * QT + qt) * KT + kt) << 10) + lane * 16);
    f32x16 sb;                                                  // the bias tile in accumulator order, once
#pragma unroll
    for (int v = 0; v < 16; ++v) sb[v] = 0.0f;
#pragma unroll
    for (int i = 0; i < NF; ++i) MM::mma(sb, ident[i], bc.frag(i));

    f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
    for (int b2 = slice; b2 < B2; b2 += NS) {
        const long bh = (long)b2 * H + h;
        const float kb = keybias[(long)b2 * KT * 32 + key];
        f32x16 s = sb, dp;
#pragma unroll
        for (int v = 0; v < 16; ++v) dp[v] = 0.0f;
#pragma unroll
        for (int p = 0; p < DP; ++p) {
            Tile16<T> qc, doc, kf, vf;
            qc.load(q_qk + p * part_q + ((bh * QT + qt) << 10) + lane * 16);
            doc.load(do_qk + p * part_q + ((bh * QT + qt) << 10) + lane * 16);
            kf.load(k_qk + p * part_k + ((bh * KT + kt) << 10) + lane * 16);
            vf.load(v_qk + p * part_k + ((bh * KT + kt) << 10) + lane * 16);
#pragma unroll
            for (int i = 0; i < NF; ++i) MM::mma(s, qc.frag(i), kf.frag(i));
#pragma unroll
            for (int i = 0; i < NF; ++i) MM::mma(dp, doc.frag(i), vf.frag(i));
        }
        const float* lp = lse + (bh * QT + qt) * 32 + 4 * half;
        const float* dpz = dsum + (bh * QT + qt) * 32 + 4 * half;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const f32x4 L4 = *reinterpret_cast<const f32x4*>(lp + 8 * g);
            const f32x4 D4 = *reinterpret_cast<const f32x4*>(dpz + 8 * g);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int v = 4 * g + e;
                acc[v] += fast_exp2(s[v] + kb - L4[e]) * (dp[v] - D4[e]);
            }
        }
    }
    if (key < Nk) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int qrow = qt * 32 + acc_row(v, lane);
            if (qrow < Nq) atomicAdd(dbias + ((long)h * Nq + qrow) * Nk + key, acc[v]);
        }
    }
}

template <typename T, int DP>
int launch_bwd(void* dq, void* dk, void* dv, float* dbias, float* lse, float* dsum, const void* q_qk, const void* q_acc,
               const void* k_qk, const void* k_acc, const void* v_qk, const void* bias_t,
               const float* keybias, const void* do_qk, const void* do_acc, const void* o_qk, long B2, long H, long Nq,
               long Nk, float dq_scale, float dk_scale, hipStream_t st) {
    const long QT = (Nq + 31) / 32, KT = (Nk + 31) / 32;
    const long part_q = B2 * H * QT * 1024, part_k = B2 * H * KT * 1024;
    const long g1 = 8 * ((B2 * H * QT + 31) / 32), g2 = 8 * ((B2 * H * KT + 31) / 32);      // blocks of four waves, a multiple of 8
    FFK_REQUIRE(g1 < (1L << 31) && g2 < (1L << 31), FFK_ERR_SHAPE, "ffk_attention_bwd: too many tiles for one launch");
    if (bias_t) {
        attention_bwd_dq_kernel<T, DP, true><<<(unsigned)g1, 256, 0, st>>>((T*)dq, lse, dsum, (const T*)q_qk, (const T*)k_qk,
                                                                         (const T*)k_acc, (const T*)v_qk, (const T*)bias_t, keybias,
                                                                         (const T*)do_qk, (const T*)o_qk, (int)B2, (int)H, (int)Nq,
                                                                         (int)Nk, dq_scale, part_q, part_k);
    } else {
        attention_bwd_dq_kernel<T, DP, false><<<(unsigned)g1, 256, 0, st>>>((T*)dq, lse, dsum, (const T*)q_qk, (const T*)k_qk,
                                                                          (const T*)k_acc, (const T*)v_qk, nullptr, keybias,
                                                                          (const T*)do_qk, (const T*)o_qk, (int)B2, (int)H, (int)Nq,
                                                                          (int)Nk, dq_scale, part_q, part_k);
    }
    int rc = ffk_check_launch("ffk_attention_bwd");
    if (rc != FFK_OK) return rc;
    attention_bwd_dkv_kernel<T, DP><<<(unsigned)g2, 256, 0, st>>>((T*)dk, (T*)dv, (const T*)q_qk, (const T*)q_acc,
                                                                (const T*)k_qk, (const T*)v_qk, (const T*)bias_t, keybias,
                                                                (const T*)do_qk, (const T*)do_acc, lse, dsum, (int)B2, (int)H,
                                                                (int)Nq, (int)Nk, dk_scale, part_q, part_k);
    rc = ffk_check_launch("ffk_attention_bwd");
    if (rc != FFK_OK || !dbias) return rc;
    // enough slices of the batch rows for ~ 8 waves per SIMD, at least 8 rows per slice
    const long tiles = H * QT * KT;
    long ns = (8L * 1024 + tiles - 1) / tiles;
    if (ns > (B2 + 7) / 8) ns = (B2 + 7) / 8;
    if (ns < 1) ns = 1;
    const long g3 = 8 * ((ns * tiles + 31) / 32);
    FFK_REQUIRE(g3 < (1L << 31), FFK_ERR_SHAPE, "ffk_attention_bwd: too many tiles for one launch");
    attention_bwd_dbias_kernel<T, DP><<<(unsigned)g3, 256, 0, st>>>(dbias, (const T*)q_qk, (const T*)k_qk, (const T*)v_qk,
                                                                  (const T*)bias_t, keybias, (const T*)do_qk, lse, dsum,
                                                                  (int)B2, (int)H, (int)Nq, (int)Nk, (int)ns, part_q, part_k);
    return ffk_check_launch("ffk_attention_bwd");
}

}  // namespace

extern "C" int ffk_attention_bwd(void* dq, void* dk, void* dv, float* dbias, float* lse, float* dsum, const void* q_qk,
                                 const void* q_acc, const void* k_qk, const void* k_acc, const void* v_qk, const void* bias_t,
                                 const float* keybias, const void* do_qk, const void* do_acc,
                                 const void* o_qk, int64_t B2, int64_t H, int64_t Nq, int64_t Nk, int64_t D, float dq_scale,
                                 float dk_scale, int dtype, void* stream) {
    FFK_REQUIRE(D == 32 || D == 64 || D == 128, FFK_ERR_SHAPE,
                "ffk_attention_bwd: head dimension %ld (32, 64 or 128; narrower heads arrive zero-padded to 32)", (long)D);
    FFK_REQUIRE(dq && dk && dv && lse && dsum && q_qk && q_acc && k_qk && k_acc && v_qk && keybias && do_qk && do_acc && o_qk,
                FFK_ERR_NULL, "ffk_attention_bwd: null pointer");
    FFK_REQUIRE(!dbias || bias_t, FFK_ERR_NULL, "ffk_attention_bwd: dbias needs bias_t");
    FFK_REQUIRE(B2 > 0 && B2 < 131072 && H > 0 && H < 65536 && Nq > 0 && Nk > 0 && Nq < (1 << 24) && Nk < (1 << 24),
                FFK_ERR_SHAPE, "ffk_attention_bwd: bad shape B2=%ld H=%ld Nq=%ld Nk=%ld", (long)B2, (long)H, (long)Nq, (long)Nk);
    FFK_REQUIRE(ffk_aligned16(dq) && ffk_aligned16(dk) && ffk_aligned16(dv) && ffk_aligned16(lse) && ffk_aligned16(dsum) &&
                    ffk_aligned16(q_qk) && ffk_aligned16(q_acc) && ffk_aligned16(k_qk) && ffk_aligned16(k_acc) &&
                    ffk_aligned16(v_qk) && ffk_aligned16(keybias) && ffk_aligned16(do_qk) && ffk_aligned16(do_acc) &&
                    ffk_aligned16(o_qk) && (!bias_t || ffk_aligned16(bias_t)),
                FFK_ERR_ALIGN, "ffk_attention_bwd: buffers must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
#define FFK_BWD_ARGS dq, dk, dv, dbias, lse, dsum, q_qk, q_acc, k_qk, k_acc, v_qk, bias_t, keybias, do_qk, do_acc, o_qk, \
                     B2, H, Nq, Nk, dq_scale, dk_scale, st
    switch (dtype) {
        case FFK_BF16:
            return D == 32 ? launch_bwd<bf16_t, 1>(FFK_BWD_ARGS)
                           : (D == 64 ? launch_bwd<bf16_t, 2>(FFK_BWD_ARGS) : launch_bwd<bf16_t, 4>(FFK_BWD_ARGS));
        case FFK_F32:
            return D == 32 ? launch_bwd<float, 1>(FFK_BWD_ARGS)
                           : (D == 64 ? launch_bwd<float, 2>(FFK_BWD_ARGS) : launch_bwd<float, 4>(FFK_BWD_ARGS));
        default: return ffk_fail(FFK_ERR_DTYPE, "ffk_attention_bwd: unsupported dtype tag %d", dtype);
    }
#undef FFK_BWD_ARGS
}
