"""float64 numpy restatements of the op-level kernels on the Evoformer hot path.

TEST INFRASTRUCTURE ONLY - never imported by the product package.

Each function cites the reference definition it restates.  Pinning (tests/test_oracle.py):
softmax / layer_norm against torch's library routines and closed-form invariants,
attention_core against an explicit per-query loop, the contractions against triple loops.
"""
import numpy as np


def fused_softmax(x, mask=None, bias=None, fill=-1e9):
    """softmax(where(mask == 0, fill, x + bias), -1).

    x [B1,B2,H,Nq,Nk]; mask [B1,B2,Nk] (0/1); bias [B1,1,H,Nq,Nk].
    Reference: kernel/triton/softmax.py:13-19 (bias added, then masked entries replaced) and
    kernel/cuda_native/csrc/softmax_cuda_kernel.cu:636-641; test oracle
    tests/test_fastnn/test_softmax.py:30-32 (additive 1e9*(mask-1): identical after exp
    whenever a row keeps at least one valid key)."""
    v = np.asarray(x, dtype=np.float64)
    if bias is not None:
        v = v + np.asarray(bias, dtype=np.float64)
    if mask is not None:
        m = np.asarray(mask, dtype=np.float64)[:, :, None, None, :]
        v = np.where(m == 0, fill, v)
    v = v - v.max(axis=-1, keepdims=True)
    e = np.exp(v)
    return e / e.sum(axis=-1, keepdims=True)


def softmax_bwd(dy, y):
    """dx = (dy - sum(y*dy)) * y   (softmax_cuda_kernel.cu:252-334)."""
    dy = np.asarray(dy, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    return (dy - (y * dy).sum(-1, keepdims=True)) * y


def layer_norm(x, gamma, beta, eps=1e-5):
    """(x - mean) * rsqrt(biased var + eps) * gamma + beta over the last dim
    (kernel/triton/layer_norm.py:7-54; kernel/layer_norm.py:19-60)."""
    x = np.asarray(x, dtype=np.float64)
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * np.asarray(gamma, np.float64) + np.asarray(beta, np.float64)


def bias_sigmod_ele(y, bias, z):
    """sigmoid(y + bias) * z   (kernel/jit/fused_ops.py:5-7)."""
    y, bias, z = (np.asarray(t, np.float64) for t in (y, bias, z))
    return 1.0 / (1.0 + np.exp(-(y + bias))) * z


def bias_dropout_add(x, bias, dropmask, residual):
    """residual + (x + bias) * dropmask, eval mode   (fused_ops.py:10-15)."""
    x, bias, dropmask, residual = (np.asarray(t, np.float64) for t in (x, bias, dropmask, residual))
    return residual + (x + bias) * dropmask


def bias_ele_dropout_residual(ab, b, g, dropout_mask, z_raw):
    """Z_raw + dropout_mask * (g * (ab + b)), eval mode   (fused_ops.py:18-22)."""
    ab, b, g, dropout_mask, z_raw = (np.asarray(t, np.float64) for t in (ab, b, g, dropout_mask, z_raw))
    return z_raw + dropout_mask * (g * (ab + b))


def attention_core(q, k, v, mask=None, bias=None, fill=-1e9):
    """softmax(q k^T / sqrt(d) + bias, masked keys -> fill) v, output [b1,b2,n,(h d)].

    q,k,v [b1,b2,h,n,d]; mask [b1,b2,n]; bias [b1,h,n,n] (4-D).
    Reference: kernel/attention_core.py:17-31 (= tests/test_fastnn/test_attention_core.py:16-31)."""
    q, k, v = (np.asarray(t, np.float64) for t in (q, k, v))
    d = q.shape[-1]
    logits = np.einsum("abhqd,abhkd->abhqk", q / np.sqrt(d), k)
    if bias is not None:
        logits = logits + np.asarray(bias, np.float64)[:, None]
    if mask is not None:
        m = np.asarray(mask, np.float64)[:, :, None, None, :]
        logits = np.where(m == 0, fill, logits)
    logits = logits - logits.max(-1, keepdims=True)
    w = np.exp(logits)
    w = w / w.sum(-1, keepdims=True)
    o = np.einsum("abhqk,abhkd->abqhd", w, v)
    return o.reshape(o.shape[:3] + (-1,))


def trimul_outgoing(a, b):
    """p[i,j,c] = sum_k a[i,k,c] b[j,k,c]   (fastnn/ops.py:400-403; nn/triangular_multiplicative_update.py:116-125)."""
    return np.einsum("ikc,jkc->ijc", np.asarray(a, np.float64), np.asarray(b, np.float64))


def trimul_incoming(a, b):
    """p[i,j,c] = sum_k a[k,i,c] b[k,j,c]   (fastnn/ops.py:529-532; nn/...update.py:141-150)."""
    return np.einsum("kic,kjc->ijc", np.asarray(a, np.float64), np.asarray(b, np.float64))


def outer_product(a, b):
    """O[i,j,d*E+e] = sum_s a[s,i,d] b[s,j,e]   (fastnn/ops.py:158-159; nn/outer_product_mean.py:52-57)."""
    o = np.einsum("sid,sje->ijde", np.asarray(a, np.float64), np.asarray(b, np.float64))
    return o.reshape(o.shape[0], o.shape[1], -1)


def linear(x, w, b=None):
    """x W^T + b   (F.linear; fastnn/ops.py:229-256)."""
    y = np.asarray(x, np.float64) @ np.asarray(w, np.float64).T
    return y if b is None else y + np.asarray(b, np.float64)
