"""Writes tests/golden/vectors.npz: small seeded inputs and the outputs that the path must produce for them.

The reference holds no golden vectors for this path (its only test draws unseeded random inputs), and its Python
is not imported here.  Expected outputs come from independent mathematics evaluated in fp64 on the CPU:
dense softmax attention softmax(Q K^T / sqrt(D) + mask) V with its log-sum-exp through the installed torch's
scaled_dot_product_attention / logsumexp, gradients through torch.autograd of that library routine, the rotary
embedding by an explicit Python loop over complex numbers, and the Ulysses exchange by an explicit index loop.
Nothing here calls the oracle under oracle/ (the oracle is checked AGAINST this file) or the HIP library.

Run from the repository root:  python tests/golden/make_vectors.py
"""
import cmath
import math
import os

import numpy as np
import torch
import torch.nn.functional as F

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.npz")


def bf16_round(x):
    return x.to(torch.bfloat16).float()


def dense(q, k, v, q_pos, k_pos, causal, do=None):
    """q [B,Sq,Hq,D], k/v [B,Sk,Hkv,D] fp32 -> O, LSE (and dQ, dK, dV) in fp64 through library SDPA."""
    q, k, v = (t.double().requires_grad_(do is not None) for t in (q, k, v))
    rep = q.shape[2] // k.shape[2]
    mask = (k_pos[None, :] <= q_pos[:, None]) if causal else torch.ones(len(q_pos), len(k_pos), dtype=torch.bool)
    qh, kh, vh = q.transpose(1, 2), k.repeat_interleave(rep, 2).transpose(1, 2), v.repeat_interleave(rep, 2).transpose(1, 2)
    o = F.scaled_dot_product_attention(qh, kh, vh, attn_mask=mask).transpose(1, 2)
    s = torch.einsum("bhqd,bhkd->bhqk", qh, kh) / math.sqrt(q.shape[-1])
    lse = torch.logsumexp(s.masked_fill(~mask, float("-inf")), dim=-1)        # [B, Hq, Sq]
    if do is None:
        return o.detach(), lse.detach()
    o.backward(do.double())
    return o.detach(), lse.detach(), q.grad, k.grad, v.grad


def main():
    out = {}
    g = torch.Generator().manual_seed(20240)
    # case A: the reference's contiguous layout, fp32, MHA, causal by global position, 4 ranks x 8 tokens
    B, H, D, W, Sl = 1, 2, 64, 4, 8
    S = W * Sl
    q, k, v = (torch.randn(B, S, H, D, generator=g) for _ in range(3))
    pos = torch.arange(S)
    o, lse = dense(q, k, v, pos, pos, True)
    out.update(a_q=q.numpy(), a_k=k.numpy(), a_v=v.numpy(), a_o=o.float().numpy(), a_lse=lse.float().numpy(), a_world=np.int64(W))
    # case B: bf16 inputs (stored as their 16-bit patterns), GQA 2/1, D=64, zig-zag over 2 ranks (4 half-chunks of 16),
    # causal, with gradients
    B, Hq, Hkv, D, W, S = 1, 2, 1, 64, 2, 64
    q, do = (bf16_round(torch.randn(B, S, Hq, D, generator=g)) for _ in range(2))
    k, v = (bf16_round(torch.randn(B, S, Hkv, D, generator=g)) for _ in range(2))
    pos = torch.arange(S)
    o, lse, dq, dk, dv = dense(q, k, v, pos, pos, True, do)
    bits = lambda t: t.to(torch.bfloat16).view(torch.int16).numpy()
    out.update(b_q=bits(q), b_k=bits(k), b_v=bits(v), b_do=bits(do), b_o=o.float().numpy(), b_lse=lse.float().numpy(),
               b_dq=dq.float().numpy(), b_dk=dk.float().numpy(), b_dv=dv.float().numpy(), b_world=np.int64(W))
    # case C: rotary embedding of a chunk that starts at position 100, adjacent pairs, theta 10000, by a Python loop
    B, S0, Sc, H, D = 1, 100, 6, 2, 16
    x = torch.randn(B, Sc, H, D, generator=g)
    y = torch.zeros_like(x, dtype=torch.float64)
    for s in range(Sc):
        for i in range(D // 2):
            ang = np.float32(S0 + s) * (np.float32(1.0) / np.float32(10000.0) ** (np.float32(2 * i) / np.float32(D)))
            w = cmath.rect(1.0, float(np.float32(ang)))
            for h in range(H):
                z = complex(float(x[0, s, h, 2 * i]), float(x[0, s, h, 2 * i + 1])) * w
                y[0, s, h, 2 * i], y[0, s, h, 2 * i + 1] = z.real, z.imag
    out.update(c_x=x.numpy(), c_y=y.float().numpy(), c_pos0=np.int64(S0))
    # case D: the Ulysses exchange (scatter heads, gather sequence) of 2 ranks by an index loop
    W, B, Sl, H, D = 2, 1, 3, 4, 2
    shards = torch.arange(W * B * Sl * H * D, dtype=torch.float32).view(W, B, Sl, H, D)
    exch = torch.zeros(W, B, W * Sl, H // W, D)
    for r in range(W):              # receiving rank = head group
        for j in range(W):          # sending rank = sequence shard
            for s in range(Sl):
                for hh in range(H // W):
                    exch[r, :, j * Sl + s, hh] = shards[j, :, s, r * (H // W) + hh]
    out.update(d_in=shards.numpy(), d_out=exch.numpy())
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
