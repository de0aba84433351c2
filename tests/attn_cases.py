"""The attention layer's forward pass restated from the oracle's pieces (fp32 GEMM restatement,
textbook attention) and numpy reshapes, following src/core/attention.c:121-430; pinned against
the reference's own layer output in test_oracle.py."""
import os

import numpy as np

from axm_format import parse_axm

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def split_heads(t, B, S, H, dk):
    """[B*S, H*dk] -> [B*H, S, dk] (ax_attn_head_interleave_qkv_split, src/core/attention/layout.c:237-253)"""
    return np.ascontiguousarray(t.reshape(B, S, H, dk).transpose(0, 2, 1, 3)).reshape(B * H, S, dk)


def merge_heads(t, B, S, H, dk):
    """[B*H, S, dk] -> [B*S, H*dk] (ax_attn_head_deinterleave, layout.c:134-148)"""
    return np.ascontiguousarray(t.reshape(B, H, S, dk).transpose(0, 2, 1, 3)).reshape(B * S, H * dk)


def mha_forward(oracle, x, w, H, causal):
    """w = (Wq, Wk, Wv, Wo, bq, bk, bv, bo) or the first four only."""
    B, S, D = x.shape
    dk = D // H
    qkv = oracle.gemm_opt(x.reshape(B * S, D), np.ascontiguousarray(np.concatenate(w[:3], axis=1)))
    if len(w) == 8:
        qkv = qkv + np.concatenate(w[4:7])
    q, k, v = (split_heads(np.ascontiguousarray(qkv[:, i * D:(i + 1) * D]), B, S, H, dk) for i in range(3))
    o, _ = oracle.sdpa(q, k, v, float(np.float32(1.0) / np.sqrt(np.float32(dk))), causal)
    out = oracle.gemm_opt(merge_heads(o, B, S, H, dk), w[3])
    if len(w) == 8:
        out = out + w[7]
    return out.reshape(B, S, D).astype(np.float32)


def fixture_model(tag):
    """(layers, parameter arrays) of tests/golden/ref_<tag>.axm"""
    layers, tensors, _ = parse_axm(open(os.path.join(GOLD, f"ref_{tag}.axm"), "rb").read())
    return layers, [np.array(t) for t in tensors]


def fixture_input(oracle, tensors, in_shape, seed):
    """The input make_golden.py drew after perturbing every 1-D parameter, from seed + 1."""
    oracle.seed(seed + 1)
    for t in tensors:
        if t.ndim == 1:
            oracle.uniform((t.shape[0],), -0.5, 0.5)
    return oracle.uniform(in_shape, -1.0, 1.0)
