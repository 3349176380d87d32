/*
 * ffk - MI355X (gfx950) kernels for the FastFold Evoformer hot path.  C ABI.
 *
 * libffk.so is libtorch-free: every entry point takes raw device pointers, explicit
 * shapes / strides, a dtype tag and a HIP stream (passed as void*), launches on that
 * stream and returns an int status (FFK_OK = 0).  The library allocates nothing and
 * keeps no state; the caller owns every buffer, scratch included.  After a non-zero
 * return ffk_last_error_string() describes the failure (thread-local).
 *
 * Each entry point names the reference interface it stands in for (paths are relative
 * to the reference repository root).
 */
#ifndef FFK_H
#define FFK_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* status codes */
enum {
    FFK_OK = 0,
    FFK_ERR_DTYPE = 1,     /* dtype tag not supported by this entry point          */
    FFK_ERR_SHAPE = 2,     /* a dimension is <= 0, too large, or violates a divisibility rule */
    FFK_ERR_NULL = 3,      /* a required pointer is NULL                           */
    FFK_ERR_ALIGN = 4,     /* a pointer / leading dimension is not 16-byte aligned */
    FFK_ERR_LAUNCH = 5,    /* hipGetLastError() reported a failure after launch    */
    FFK_ERR_UNSUPPORTED = 6
};

/* element types of activation / weight buffers */
enum { FFK_F32 = 0, FFK_BF16 = 1, FFK_F16 = 2 };

int ffk_version(void);
const char* ffk_last_error_string(void);

/* ------------------------------------------------------------------------------------
 * Fused softmax:  out = softmax(where(mask == 0, -1e9, x + bias), dim = -1)
 *   x, out : [B1, B2, H, Nq, Nk]   (out may alias x: the reference's CUDA path is in place)
 *   mask   : [B1, B2, Nk] of the same dtype holding 0/1, or NULL
 *   bias   : [B1, 1, H, Nq, Nk] of the same dtype, or NULL (requires mask != NULL is NOT
 *            demanded; any combination is accepted)
 * fp32 arithmetic inside; dtype f32 / bf16 / f16.
 * Replaces: fastfold_softmax_cuda.{forward, fused_mask_softmax_forward,
 *   fused_mask_bias_softmax_forward}
 *   (fastfold/model/fastnn/kernel/cuda_native/csrc/softmax_cuda.cpp:3-27,
 *    softmax_cuda_kernel.cu:163-250,425-522,708-810) and the Triton wrapper
 *   (kernel/triton/softmax.py:153-186).
 */
int ffk_softmax_fwd(void* out, const void* x, const void* mask, const void* bias,
                    int64_t B1, int64_t B2, int64_t H, int64_t Nq, int64_t Nk,
                    int dtype, void* stream);

/* Softmax backward: dx = (dy - sum(y * dy)) * y over rows of length cols.
 * Replaces: fastfold_softmax_cuda.{backward, fused_mask_softmax_backward,
 *   fused_mask_bias_softmax_backward} (softmax_cuda_kernel.cu:252-334,524-614,812-839);
 * masked entries have y == 0 and therefore dx == 0 without consulting the mask. */
int ffk_softmax_bwd(void* dx, const void* dy, const void* y, int64_t rows, int64_t cols,
                    int dtype, void* stream);

/* Measurement aid with no counterpart in the reference: a plain streaming copy of `bytes` (a multiple of 16) with the
 * access pattern of the row kernels (16-byte non-temporal loads and stores, a grid like theirs).  bench.py times it
 * beside the fused softmax and LayerNorm: it is what a read-once / write-once stream of the same size reaches on the
 * GPU at hand, the practical ceiling of an HBM-bound row kernel. */
int ffk_stream_copy(void* dst, const void* src, int64_t bytes, void* stream);

/* ------------------------------------------------------------------------------------
 * LayerNorm over the last dimension, affine:  out = (x - mean) * rsqrt(var + eps) * gamma + beta
 *   x, out : [rows, cols] contiguous;  gamma, beta : [cols] of the same dtype
 *   mean, rstd : optional fp32 [rows] outputs (NULL to skip)
 * Replaces: fastfold_layer_norm_cuda.forward_affine
 *   (kernel/cuda_native/csrc/layer_norm_cuda.cpp:70-95, layer_norm_cuda_kernel.cu:61-152)
 *   and kernel/triton/layer_norm.py:146-176.
 */
int ffk_layernorm_fwd(void* out, float* mean, float* rstd, const void* x, const void* gamma,
                      const void* beta, int64_t rows, int64_t cols, float eps, int dtype,
                      void* stream);

/* LayerNorm backward (dx, dgamma, dbeta).  dgamma/dbeta are fp32 [cols] and must be
 * zero-filled by the caller (the kernel accumulates with atomics).
 * Replaces: fastfold_layer_norm_cuda.backward_affine (layer_norm_cuda.cpp:97-125,
 *   layer_norm_cuda_kernel.cu:224-500). */
int ffk_layernorm_bwd(void* dx, float* dgamma, float* dbeta, const void* dy, const void* x,
                      const float* mean, const float* rstd, const void* gamma,
                      int64_t rows, int64_t cols, int dtype, void* stream);

/* ------------------------------------------------------------------------------------
 * Elementwise fusions (eval-mode dropout: the mask tensor multiplies as given).
 * Tensors are viewed as [B, I, J, C]; `dm` is the dropout mask with strides (in elements)
 * dm_sb, dm_si, dm_sj for the first three axes (0 = broadcast) and unit stride on C;
 * dm may be NULL (= all ones).
 *   ffk_bias_sigmoid_mul      : out = sigmoid(y + bias[C]) * z
 *   ffk_bias_dropout_add      : out = residual + (x + bias[C]) * dm
 *   ffk_bias_ele_dropout_res  : out = z_raw + dm * (g * (ab + bias[C]))
 * Replaces: bias_sigmod_ele, bias_dropout_add, bias_ele_dropout_residual
 *   (fastfold/model/fastnn/kernel/jit/fused_ops.py:5-22).
 */
int ffk_bias_sigmoid_mul(void* out, const void* y, const void* bias, const void* z,
                         int64_t rows, int64_t C, int dtype, void* stream);
int ffk_bias_dropout_add(void* out, const void* x, const void* bias, const void* dm,
                         const void* residual, int64_t B, int64_t I, int64_t J, int64_t C,
                         int64_t dm_sb, int64_t dm_si, int64_t dm_sj, int dtype, void* stream);
int ffk_bias_ele_dropout_res(void* out, const void* ab, const void* bias, const void* g,
                             const void* dm, const void* z_raw, int64_t B, int64_t I, int64_t J,
                             int64_t C, int64_t dm_sb, int64_t dm_si, int64_t dm_sj, int dtype,
                             void* stream);


/* ------------------------------------------------------------------------------------
 * Extended residual stream.  A 48-block bf16 stack adds about 300 updates to each of its two activation tensors;
 * rounding the sum to bf16 after every one of them is a random walk of half-ulp errors that ends near 2e-2 relative,
 * above the tolerance of the bf16 mode.  Every entry point that adds an update to such a tensor (`resid`) therefore
 * accepts an optional tail tensor of signed bytes with the same shape: the pair (h, t) of a bf16 element and its tail
 * byte stands for the fp32 bit pattern (bits(h) << 16) + (t << 8), i.e. eight more mantissa bits, h being that value
 * rounded to bf16 - a reader that ignores the tail sees an ordinary, correctly rounded bf16 tensor.  The tail is
 * read and rewritten in place (a zero-filled tail is an exact bf16 tensor; dropping the tails at the end leaves the
 * correctly rounded result), bf16 only.  No counterpart in the reference, which keeps the plain bf16 stream. */

/* ------------------------------------------------------------------------------------
 * Fused linear:  out = epilogue( prologue(A)[M,K] . W[N,K]^T )      (bf16 / fp32 MFMA)
 *
 * A tile of rows of A (all K columns, K in {32..256}, K % 32 == 0) is loaded into LDS once,
 * optionally LayerNorm-ed there (gamma/beta over K), and then multiplied against every
 * 128-row tile of W; each such N-tile has its own epilogue descriptor, so one pass over
 * A feeds several consumers (q, k, v, gate, bias projections of one attention, or the
 * gated left/right projections of a triangle multiplication).
 *
 * Row addressing.  Logical row m of A lives at  a + (m / a_inner) * a_so + (m % a_inner) * a_si
 * (elements; K is contiguous), which expresses plain row-major ([M,K]: a_inner = M) as well as
 * the transposed traversals of [I,J,C] tensors used by column-wise modules.  With
 * a_chanmajor != 0 element (m, k) lives at  a + k * a_cs + rowoffset(m)  instead (channel-major
 * producer, e.g. the triangle contraction output).  Output tiles use the same scheme with
 * (s_o, s_i) for rows and  (c / 32) * s_h + (c % 32) * s_d  for channel c of the tile.
 *
 * Tile kinds:
 *   FFK_TILE_STRIDED  generic 4-stride store; optional  out = resid + gate * v
 *   FFK_TILE_QK       q / k of attention in MFMA-operand tiles: [b2][h][n/32][d/16][n%32][d%16]
 *   FFK_TILE_V        v of attention in PV-operand tiles (see ffk_attention_fwd)
 *   FFK_TILE_BIAS     pair / triangle bias in score-accumulator tiles (see ffk_attention_fwd)
 *                     (as the LAST tile of a bf16, K = 128 launch with <= 4 channels it takes no weight slot: the
 *                     weights-stationary kernel computes it with 16 x 16 x 32 MFMAs from the rows it holds in LDS)
 *   FFK_TILE_ACC      [b2][h][n/32] tiles in MFMA accumulator order: element (n, d) of a tile at
 *                     ((d & 7) >> 2) * 512 + (n % 32) * 16 + 4 * (d >> 3) + (d & 3), i.e. the lane that
 *                     owns row n in a 32x32 accumulator holds its 16 channels contiguously.  Valid for
 *                     q and k (any common order of the head dim gives the same q.k) and required
 *                     for a gate that ffk_attention_fwd reads with FFK_ATT_GATE_TILED.
 * Per-tile value: v = act(acc + bias[c]) * scale; with glu != 0 the tile's packed channels are
 * [p 0..31 | g 0..31 | p 32..63 | g 32..63] and v = (p + bias_p) * sigmoid(g + bias_g) (64
 * outputs); rowmask (0/1 per logical row, own strides) multiplies v.
 *
 * Replaces the F.linear + LayerNorm + elementwise chains of fastfold/model/fastnn/ops.py:
 * 79-82,143-155,305-324,393-399,404-412,659-670 and msa.py:61-72.
 */
enum { FFK_TILE_STRIDED = 0, FFK_TILE_QK = 1, FFK_TILE_V = 2, FFK_TILE_BIAS = 3, FFK_TILE_ACC = 4 };
enum { FFK_ACT_NONE = 0, FFK_ACT_RELU = 1, FFK_ACT_SIGMOID = 2 };
enum { FFK_LINEAR_AUTO = 0, FFK_LINEAR_STAGED = 1 };
#define FFK_MAX_TILES 10

typedef struct ffk_tile {
    void* out;
    const void* bias;      /* 128 values of the activation dtype (packed tile order) or NULL */
    const void* resid;     /* same addressing as out (may alias out) or NULL; STRIDED with s_d == 1 only */
    const void* gate;      /* [M, gate_ld] in logical row order (gate_rows == 0) or [gate_rows, gate_ld] read at
                              row m % gate_rows (one multiplier row shared by every gate_rows-th logical row),
                              or NULL; STRIDED with s_d == 1 only */
    const void* rowmask;   /* 0/1 per logical row at (m / inner) * m_so + (m % inner) * m_si, or NULL */
    int64_t s_o, s_i, s_h, s_d;
    int64_t gate_ld;
    int64_t m_so, m_si;
    int32_t inner;
    int32_t kind;
    int32_t act;
    int32_t ncols;         /* valid output channels of this tile (<= 128, <= 64 with glu) */
    int32_t glu;
    float scale;
    int32_t gate_rows;     /* 0, or the period of the gate's row index (see gate) */
    int32_t reserved;
    void* xtail;           /* NULL, or the tail bytes of an extended residual stream (see above): int8, addressed with
                              the element offsets of out; requires resid (bf16, STRIDED with s_d == 1).  The epilogue then
                              adds its update to the 24-bit value (resid, xtail), writes the rounded bf16 value to out and
                              the new tail back to xtail */
} ffk_tile;

typedef struct ffk_linear_desc {
    const void* a;
    int64_t a_so, a_si, a_cs;
    int32_t a_inner;
    int32_t a_chanmajor;
    const void* ln_gamma;  /* NULL = no LayerNorm prologue */
    const void* ln_beta;
    float ln_eps;
    int32_t dtype;
    const void* w;         /* [n_tiles * 128, K] row-major, zero-padded rows */
    int32_t M, K, n_tiles;
    /* ln_folded: 0, or 1 together with a second operand (a2, below): LayerNorms are then not applied to the
       rows but folded into the weights.  For a row x of either operand with statistics (mean, rstd),
           W LN(x) + b = rstd * (W' x - mean * rowsum(W')) + b',   W' = W * gamma,  b' = W beta + b,
       so w holds W' (value rows: the first operand's gamma, gate rows: the second operand's), the tile
       biases hold b', ln_gamma points to an fp32 table [n_tiles * 128] of the row sums of W' in packed tile
       order and ln_beta / ln2_gamma / ln2_beta are ignored; the kernel takes mean and rstd of a row from the
       operand fragments it multiplies anyway.  Tiles must be plain residual GLU tiles of 64 channels (no
       gate pointer, no row mask, scale 1). */
    int32_t ln_folded;
    /* Optional second operand (NULL = none): the gate halves of the GLU tiles are then computed from
       LayerNorm(a2) instead of from the first operand, both LayerNorms folded into the weights (ln_folded must
       be 1).  a2 is K-contiguous, logical row m at  a2 + (m / a2_inner) * a2_so + (m % a2_inner) * a2_si.
       Built for bf16, K = 128 and a channel-major first operand (the output stage of the triangle
       multiplication, whose gate comes from the pair tensor and whose value from the contraction result);
       other combinations return FFK_ERR_UNSUPPORTED. */
    const void* a2;
    const void* ln2_gamma;
    const void* ln2_beta;
    int64_t a2_so, a2_si;
    int32_t a2_inner;
    int32_t variant;       /* FFK_LINEAR_AUTO, or FFK_LINEAR_STAGED to force the LDS-staged kernels (used by tests that
                              compare the kernel variants with each other) */
    ffk_tile tiles[FFK_MAX_TILES];
} ffk_linear_desc;

int ffk_fused_linear(const ffk_linear_desc* desc, void* stream);


/* ------------------------------------------------------------------------------------
 * Batched "NT" GEMM with a K loop:  C[b] = epilogue( A[b][M,K] . B[b][N,K]^T )
 *
 * Both operands are K-contiguous (row strides lda / ldb, batch strides a_bs / b_bs, all in
 * elements; K % 8 == 0 for bf16, % 4 for fp32; rows 16-byte aligned).  The epilogue computes
 *     v = act(acc + bias[n]) * scale ;  v /= (rowdiv[m] + div_eps) ;  v += resid[m, n]
 * and stores element (m, n) of batch b at
 *     out + b * o_bs + (m / inner) * s_o + (m % inner) * s_i + (n / 32) * s_h + (n % 32) * s_d.
 * out_f32 != 0 stores fp32 regardless of the operand dtype (used for the outer-product-mean
 * normaliser).  resid uses the output addressing and may alias out.
 *
 * Used for: the triangle-multiplication contraction p[c,i,j] = sum_k l[c,i,k] r[c,j,k]
 * (torch.matmul of permuted operands, fastfold/model/fastnn/ops.py:400-403,529-532), the
 * outer-product-mean einsum and its output projection (ops.py:152,158-161,173) and the second
 * linear of the transitions (ops.py:81,96).
 */
typedef struct ffk_bgemm_desc {
    const void* a;
    const void* b;
    void* out;
    const void* bias;      /* [N] operand dtype, or NULL */
    const void* resid;     /* or NULL */
    const float* rowdiv;   /* fp32 [M] (per batch: + b * M), or NULL */
    void* xtail;           /* NULL, or the tail bytes of resid / out as an extended residual stream (bf16, s_d == 1) */
    int64_t lda, ldb, a_bs, b_bs, o_bs;
    int64_t s_o, s_i, s_h, s_d;
    int32_t inner;
    int32_t M, N, K, batch;
    int32_t dtype, act, out_f32;
    float scale, div_eps;
} ffk_bgemm_desc;

int ffk_bgemm_nt(const ffk_bgemm_desc* desc, void* stream);


/* ------------------------------------------------------------------------------------
 * Flash-style attention core (logits never reach HBM) for head dimension D = 32 - the Evoformer's, and the tuned
 * path - and D = 64 / 128, the other widths the reference's kernel accepts (kernel/triton/attention_core.py:142):
 *     o[b2, q, h, :] = softmax_k( q.k^T + bias[h, q, k] + keybias[b2, k] ) . v   (* gate)
 * in the exp2 domain: q must already carry the factor  d^-1/2 * log2(e)  and bias the
 * factor log2(e); keybias is fp32 (0 for a valid key, -1e9*log2e for a masked key and a
 * hugely negative finite value for the padding up to a multiple of 32; build it with
 * ffk_key_bias).  Operands arrive in 32x32 operand tiles (1024 elements, see
 * ffk_fused_linear tile kinds):
 *   q_t, k_t : [B2][H][ceil(N/32)][1024]   FFK_TILE_QK or FFK_TILE_ACC order (the same for both)
 *   v_t      : [B2][H][ceil(Nk/32)][1024]  FFK_TILE_V  order
 *   bias_t   : [H][ceil(Nq/32)][ceil(Nk/32)][1024]  FFK_TILE_BIAS order (keys x queries as an
 *              MFMA operand: element (k, q) at (q%32/16)*512 + (k%32)*16 + q%16), or NULL; with
 *              FFK_ATT_BIAS_PADDED in flags [H][ceil(Nq/32)][ceil(Nk/32) + 1][1024]: one unused tile ends every
 *              query-tile row, so that rows of 2^n key tiles do not start in the same memory channel (D = 32 only)
 *   keybias  : [B2][ceil(Nk/32)*32] fp32
 *   FFK_ATT_HALF_K in flags (D = 32 only): the caller guarantees that elements 8 .. 15 of every lane's sixteen (elements
 *              16 l + 8 .. 16 l + 15 of each 1024-element q and k tile) are zero - zero-padded heads of at most 16 channels
 *              in FFK_TILE_ACC order (channels 16 .. 31), of at most 8 channels in FFK_TILE_QK order (channels 8 .. 15 and
 *              24 .. 31) -; the kernel skips that half of the score product
 *   tileflags: [B2][ceil(Nk/32)] int32 per 32-key tile: 0 all keys valid, 1 mixed, 2 all masked
 *   gate     : multiplicative gate (already sigmoid-ed) or NULL: [B2*Nq, H*32] row-major, or with
 *              FFK_ATT_GATE_TILED in flags [B2][H][ceil(Nq/32)][1024] in FFK_TILE_ACC order
 *   out      : [B2*Nq, H*D] row-major
 * D = 64 / 128: the head is cut into D / 32 parts of 32 channels; q_t, k_t (FFK_TILE_QK order) and v_t hold one
 * [B2][H][ceil(N/32)][1024] block per part, part-major ([D/32][B2][H][...]: part p = channels 32p .. 32p+31 of
 * every head), q still carries d^-1/2 * log2(e) with d = D; gate must be NULL.
 * Replaces: the matmul / fused_softmax / matmul (+ bias_sigmod_ele) chain of
 * SelfAttention.forward (fastfold/model/fastnn/ops.py:310-322) and
 * fused_attention_core (kernel/attention_core.py:17-52, kernel/triton/attention_core.py:12-190).
 */
enum { FFK_ATT_GATE_TILED = 1, FFK_ATT_BIAS_PADDED = 2, FFK_ATT_HALF_K = 4 };
int ffk_attention_fwd(void* out, const void* q_t, const void* k_t, const void* v_t,
                      const void* bias_t, const float* keybias, const int32_t* tileflags, const void* gate,
                      int64_t B2, int64_t H, int64_t Nq, int64_t Nk, int64_t D, int flags, int dtype, void* stream);

/* Backward of ffk_attention_fwd without a gate (the autograd path of fused_attention_core):
 *     given do = d loss / d out, computes dq, dk, dv and (optionally) dbias of
 *     out[b2, q, h, :] = softmax_k( q.k / sqrt(d) + bias[h, q, k] + keybias[b2, k] ) . v
 * with the logits recomputed tile by tile (nothing of size Nq x Nk is stored except dbias).  Operands come in the
 * 32 x 32 tile orders of ffk_attention_fwd, each in the order(s) its roles need:
 *   q_qk, q_acc : q scaled by log2(e) / sqrt(d), [B2][H][ceil(Nq/32)][1024] in FFK_TILE_QK and in FFK_TILE_V order
 *   k_qk, k_acc : k, [B2][H][ceil(Nk/32)][1024] in FFK_TILE_QK and in FFK_TILE_V order
 *   v_qk        : v in FFK_TILE_QK order
 *   do_qk, do_acc, o_qk : do and the forward output, as [B2][H][Nq][32] tensors tiled like q
 *   bias_t      : bias * log2(e) in FFK_TILE_BIAS order, or NULL
 *   keybias     : as for ffk_attention_fwd
 *   lse, dsum   : fp32 scratch [B2][H][ceil(Nq/32)*32] (row log-sum-exp in the log2 domain and sum_d do.o; written by
 *                 the first kernel, read by the second)
 *   D = 64 / 128: every tiled operand part-major as for ffk_attention_fwd ([D/32] blocks of the D = 32 layout)
 *   dq : [B2][H][Nq][D], dk, dv : [B2][H][Nk][D] (operand dtype);  dbias : fp32 [H][Nq][Nk], ZEROED by the caller:
 *                 a third kernel sums dS over slices of the batch rows in registers and adds each slice's sum with
 *                 one atomic per element (summation order across slices not fixed), or NULL
 *   dq_scale = 1 / sqrt(d), dk_scale = 1 / log2(e): undo the factors folded into the q operand.
 * Rows whose keys are all masked get zero gradients (the forward pass gives them zero output).
 * Replaces: autograd through the matmul / fused_softmax / matmul chain of SelfAttention.forward
 * (fastfold/model/fastnn/ops.py:310-322; softmax backward kernels softmax_cuda_kernel.cu:252-334,524-614). */
int ffk_attention_bwd(void* dq, void* dk, void* dv, float* dbias, float* lse, float* dsum, const void* q_qk,
                      const void* q_acc, const void* k_qk, const void* k_acc, const void* v_qk, const void* bias_t,
                      const float* keybias, const void* do_qk, const void* do_acc,
                      const void* o_qk, int64_t B2, int64_t H, int64_t Nq, int64_t Nk, int64_t D, float dq_scale,
                      float dk_scale, int dtype, void* stream);

/* Re-tiles a strided tensor x[b2, h, n, d] (element at src + b2*s_b + h*s_h + n*s_n + d, strides in elements,
 * d contiguous, D <= 32) into [B2][H][ceil(N/32)][1024] operand tiles of ffk_attention_fwd / ffk_attention_bwd, in
 * FFK_TILE_QK or FFK_TILE_V order: rows past N and channels past D are zero, and every element is multiplied by
 * `scale` in fp32 before it is rounded (the log2(e) / sqrt(d) of the q operand; 1 for the others).
 * Replaces: the rearrange / transpose / contiguous chain in front of the reference's attention kernels
 * (fastfold/model/fastnn/ops.py:303-306; kernel/attention_core.py:24-31), which here has to end in tile order. */
int ffk_tile_pack(void* dst, const void* src, int64_t B2, int64_t H, int64_t N, int64_t D, int64_t s_b, int64_t s_h,
                  int64_t s_n, float scale, int kind, int dtype, void* stream);

/* Batched 2-D transposition with strides (all strides in elements):
 *     out[b][y][x] = in[b][x][y]      for b < B, x < X, y < Y,
 * in element (b, x, y) at in + b*in_bs + x*in_xs + y (y contiguous), out element (b, y, x) at
 * out + b*out_bs + y*out_ys + x (x contiguous); elements of 2 bytes (FFK_BF16, FFK_F16) or 4 bytes (FFK_F32).  Bytes
 * of out that no (b, y, x) addresses (padding columns) are left as they are.  out and in must not overlap.
 * Replaces: the permute_final_dims(...) + contiguous copies in front of the batched matmuls of the triangle
 * multiplications and of their backward passes (fastfold/model/fastnn/ops.py:400-403, 529-532). */
int ffk_transpose_batched(void* out, const void* in, int64_t B, int64_t X, int64_t Y, int64_t in_bs, int64_t in_xs,
                          int64_t out_bs, int64_t out_ys, int dtype, void* stream);

/* Pair bias of a biased attention, straight into the operand tiles ffk_attention_fwd reads:
 *     bias_t[h][q/32][k/32][tile(k, q)] = scale * ( LayerNorm(z[q, k, :]; gamma, beta, eps) . w[h, :] )
 * z holds N*N rows of C channels; logical row m = q*N + k lives at (m / a_inner) * a_so + (m % a_inner) * a_si
 * (elements), which also expresses the transposed traversal of the ending-node attention.
 * w is [H][C], H <= 8; bias_t is [H][ceil(N/32)][ceil(N/32)][1024] in FFK_TILE_BIAS order and must be
 * zero-filled by the caller when N is not a multiple of 32; scratch is caller-owned device memory of
 * at least 16*C + 16 floats (the kernel builds its weight operand there; with w == NULL it uses the
 * operand a previous call with the same w, gamma, beta and scratch left there, gamma / beta may then be
 * NULL too).  bf16, C = 128 or 64.
 * Replaces: F.linear(LayerNorm(Z), linear_b_weights) and its permute / unsqueeze
 * (fastfold/model/fastnn/msa.py:61-66, ops.py:659-664,890-896). */
int ffk_pair_bias(void* bias_t, const void* z, const void* gamma, const void* beta, const void* w,
                  float* scratch, int64_t N, int64_t C, int64_t H, int64_t a_inner, int64_t a_so,
                  int64_t a_si, float scale, float eps, int dtype, void* stream);

/* ffk_pair_bias for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): same arguments and results, without the scratch argument.  It has no
 * counterpart in the reference.  The weight operand is built in a 8 256-byte array that the library holds in each
 * GPU's memory for the life of the process (C <= 128 channels, H <= 8 heads; larger values are rejected with
 * FFK_ERR_SHAPE).  The call allocates and frees nothing.  w, gamma and beta are required: every call rebuilds the
 * operand, because all calls on one GPU share that GPU's array - calls that overlap on one GPU (different streams
 * or host threads) race on it and must be serialised by the caller. */
int ffk_pair_bias_static(void* bias_t, const void* z, const void* gamma, const void* beta, const void* w,
                         int64_t N, int64_t C, int64_t H, int64_t a_inner, int64_t a_so, int64_t a_si,
                         float scale, float eps, int dtype, void* stream);

/* Fused core of the outer-product-mean (bf16, 32 projected channels, 128 pair channels):
 *     out[i, j, c] = resid[i, j, c] + ( sum_{d,e} (sum_s a[s,i,d] b[s,j,e]) * w[c, d, e] + bias[c] ) / (norm[i, j] + eps)
 * a_t, b_t : [r*32, spad] the masked projections, transposed (row i*32 + d, K = sequences, zero padded
 *            to spad = 64 or 128); w2p : [128, 1024] with column e*32 + d (the reference weight has d*32 + e);
 * norm : fp32 [r, r]; resid / out : [r*r, 128] (may alias); xtail : NULL or the [r*r, 128] tail bytes of
 * resid / out as an extended residual stream; r % 32 == 0.
 * The [r, r, 1024] outer product is never written to memory.
 * Replaces: the einsum / o_linear / division chain of OutProductMean.forward
 * (fastfold/model/fastnn/ops.py:156-171; nn/outer_product_mean.py:93-127). */
int ffk_opm_fused(void* out, const void* resid, void* xtail, const void* a_t, const void* b_t, const void* w2p,
                  const void* bias, const float* norm, int64_t r, int64_t spad, float eps, int dtype,
                  void* stream);

/* Fused transition (bf16; C = 128 with hidden = 512: pair transition, C = 256 with hidden = 1024: MSA transition):
 *     out = x + W2 . relu( W1 . LayerNorm(x; gamma, beta, eps) + b1 ) + b2
 * x, out : [M, C] row-major (may alias); xtail : NULL or the [M, C] tail bytes of x / out as an extended residual
 * stream (the LayerNorm reads x alone); w1 : [hidden, C]; w2 : [C, hidden]; b1 : [hidden]; b2 : [C].
 * The hidden activation never leaves the chip.
 * Replaces: Transition.forward / ChunkTransition.forward (fastfold/model/fastnn/ops.py:79-82,104-123). */
int ffk_transition_fused(void* out, const void* x, void* xtail, const void* gamma, const void* beta, const void* w1,
                         const void* b1, const void* w2, const void* b2, int64_t M, int64_t C,
                         int64_t hidden, float eps, int dtype, void* stream);

/* Gated output stage of a gated attention (bf16; C = 128 or 256 channels, H * 32 = C gate channels):
 *     out[row m] = x[row m] + Wo . ( sigmoid( Wg . LayerNorm(x[row m]; gamma, beta, eps) + bg ) * o[m] ) + bo
 * x, out : the tensor the attention updates, logical row m at (m / inner) * s_o + (m % inner) * s_i (elements, C
 * contiguous channels; may alias); o : [M, C] the heads' weighted averages in logical row order (ffk_attention_fwd
 * called without a gate); wg : [C, C] gate projection, bg : [C]; wo : [C, C] output projection, bo : [C] or NULL;
 * xtail : NULL or the tail bytes of x / out as an extended residual stream (addressed like x).
 * The gate is computed where it is used: it is neither written by the projection launch nor read by the attention
 * core.  Replaces: gating_linear + bias_sigmod_ele + o_linear (+ bias_dropout_add in eval mode) of
 * SelfAttention.forward and its callers (fastfold/model/fastnn/ops.py:320-324, 666-670; msa.py:66-72,96-100). */
int ffk_gated_out_fused(void* out, const void* x, void* xtail, const void* gamma, const void* beta, const void* wg,
                        const void* bg, const void* o, const void* wo, const void* bo, int64_t M, int64_t C,
                        int64_t inner, int64_t s_o, int64_t s_i, float eps, int dtype, void* stream);

/* Global column attention core of the extra-MSA stack: one query per residue column (the masked mean
 * of the normalised rows), one key / value head of width D shared by the H query heads.
 *     x_s = LayerNorm(m[s, j, :]; gamma, beta, ln_eps)
 *     q[h] = scaling * Wq[h] (sum_s mask[s, j] x_s / (sum_s mask[s, j] + eps))
 *     o[j, h*D + d] = sum_s softmax_s(q[h] . Wk x_s, masked s replaced by -1e9) (Wv x_s)[d]
 * Row (s, j) of m lives at  m + s * m_ss + j * m_sr  (elements; its C channels, C in {32, 64, 128},
 * contiguous), mask[s, j] (activation dtype, 0 / 1; NULL = all ones) at  mask + s * mask_ss + j * mask_sr.
 * ln_gamma == NULL: the rows are taken as already normalised.
 * wq : [H*D, C]; wk, wv : [D, C]; o : [R, H*D]; H <= 8, H*D <= 128.  fp32 or bf16; the sums run in
 * fp32.  A column whose rows are all masked gets the plain mean of v (the softmax of equal logits),
 * as in the reference.
 * Replaces: LayerNorm + the q / k / v / softmax / weighted-average part of GlobalAttention.forward
 * (fastfold/model/fastnn/ops.py:1006-1009,1179-1195; nn/primitives.py:452-486). */
int ffk_global_attention_core(void* o, const void* m, const void* mask, const void* ln_gamma,
                              const void* ln_beta, float ln_eps, const void* wq, const void* wk,
                              const void* wv, int64_t S, int64_t R, int64_t C, int64_t H, int64_t D,
                              int64_t m_ss, int64_t m_sr, int64_t mask_ss, int64_t mask_sr,
                              float scaling, float eps, int dtype, void* stream);

/* Pair-representation part of the input embedder and of the recycling embedder:
 *     out[i, j, :] = [LayerNorm(z[i, j, :])] + table[bin(i, j), :] + [bias] + [row[i, :]] + [col[j, :]]
 * (terms in brackets are skipped when their pointer is NULL; a pair that falls in no bin gets no table row).
 * A Linear applied to a one-hot vector picks one column of its weight: `table` is that weight transposed,
 * [nb, C], and the one-hot tensor is never formed.
 *   FFK_EMBED_RELPOS     pos : [r] residue indices (fp32); bin = nearest of the offsets -k .. k (nb = 2k + 1)
 *                        to pos[i] - pos[j], the lower one on a tie
 *   FFK_EMBED_DISTOGRAM  pos : [r, 3] coordinates (fp32); edges : [nb] squared lower bin edges (fp32);
 *                        bin = the b with edges[b] < |pos_i - pos_j|^2 < edges[b + 1] (inf after the last),
 *                        open intervals as in the reference: a distance on an edge is in no bin
 * out, z : [r, r, C] (may alias), C in {64, 128, 256}; row, col : [r, C]; fp32 or bf16.
 * Replaces: InputEmbedder.forward's relpos / one_hot / linear_relpos / broadcast adds and
 * RecyclingEmbedder.forward's distogram one-hot / linear / layer_norm_z
 * (fastfold/model/fastnn/ops.py:1306-1324, 1108-1145; nn/embedders.py:82-127, 208-230). */
enum { FFK_EMBED_RELPOS = 0, FFK_EMBED_DISTOGRAM = 1 };
int ffk_pair_embed(void* out, const void* z, const void* ln_gamma, const void* ln_beta, float ln_eps,
                   const void* table, const void* bias, const void* row, const void* col, int mode,
                   const float* pos, const float* edges, float inf, int64_t r, int64_t C, int64_t nb,
                   int dtype, void* stream);

/* Attention of every position over its own short list of key / value rows (template point-wise attention):
 *     w[p, h, t] = softmax_t( q[p, h, :] . k[t, p, h, :] + bias[t] ),   o[p, h, :] = sum_t w[p, h, t] v[t, p, h, :]
 * q, o : [P, H * D] (q already scaled by 1 / sqrt(D)); kv : row (t, p) starts at kv + t * kv_st + p * kv_sp
 * (elements) and holds the H * D key channels at offset 0 and the H * D value channels at offset v_off;
 * bias : [NT] fp32 (inf * (template_mask - 1)); out_scale : NULL or one fp32 value on the device that multiplies
 * o (0 when no template is valid: the reference zeroes the update then); 1 <= NT <= 8; D in {8, 16, 32}; fp32 or bf16.
 * Replaces: the softmax(q k^T + bias) v core of TemplatePointwiseAttention.forward, where the reference calls
 * its generic Attention module on a [N_res, N_res, 1, C_z] query and [N_res, N_res, N_templ, C_t] keys
 * (fastfold/model/fastnn/template.py:83-131; nn/template.py:95-133; nn/primitives.py:344-419). */
int ffk_pointwise_attention_core(void* o, const void* q, const void* kv, const float* bias, const float* out_scale,
                                 int64_t P, int64_t H, int64_t D, int64_t NT, int64_t kv_st, int64_t kv_sp, int64_t v_off,
                                 int dtype, void* stream);

/* keybias[b, k] = mask[b, k] != 0 ? 0 : -1e9*log2(e) for k < N, and -3e38 for N <= k < Npad
 * (Npad = ceil(N/32)*32).  mask is [B, N] with strides (mask_sb, mask_sn) in elements of the
 * given dtype, or NULL (all keys valid).  tileflags[b, k/32] classifies each 32-key tile (see
 * ffk_attention_fwd).  Replaces the `1e9 * (mask - 1)` key-padding term of
 * the reference (ops.py:313, kernel/triton/softmax.py:17-19). */
int ffk_key_bias(float* keybias, int32_t* tileflags, const void* mask, int64_t B, int64_t N,
                 int64_t mask_sb, int64_t mask_sn, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FFK_H */
