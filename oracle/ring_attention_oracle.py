"""CPU oracle for the context-parallel ring / Ulysses attention path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this module; only
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do,
and only as the checker (or as the timed CPU baseline), never as the thing shipped.

It restates, in eager PyTorch on the CPU, the composition that the reference builds
from ``torch.matmul/exp/max/sum``:

* ``ring_attention_recurrence``  follows  parallel/communication/ring_attention.py:20-28
  (scale, state init), :66-107 (score GEMM, block-local-max online softmax, PV GEMM,
  output rescale) and :118 (final normalise), visiting KV chunks in the order fixed by
  :39-60 / :110-115 (rank r sees chunks r, r-1, r-2, ... mod W -> ``ring_order``).
* ``seq_all_to_all`` follows parallel/parallel_cp.py:49-73 (split on scatter_dim,
  exchange, cat on gather_dim) for ALL ranks at once, with the exchange done by
  indexing; the backward of :75-96 is the same call with the two dims swapped.
* ``precompute_freqs_cis`` / ``apply_rotary_emb`` follow layers/layers.py:18-24 and
  :44-70 (adjacent-pair complex rotation in fp32, cast back to the input dtype).
* ``kv_head_of`` follows model/model.py:11-34 (repeat_kv: consecutive repetition).
* ``contiguous_positions`` follows data/dataloader.py:156-171 (rank r owns tokens
  [r*S_l, (r+1)*S_l)).

What the reference does NOT contain and the oracle therefore defines by closed form
(dense softmax attention and its gradient): causal masking by global position inside
the ring, the log-sum-exp output, the backward pass, GQA inside the ring, the zig-zag
chunk assignment, and the (O, LSE) pair merge.

Pinning (see tests/test_oracle.py): every function here is checked against something
that is not a retyping of its own formula - torch's scaled_dot_product_attention in
fp64, pure-Python brute force on tiny inputs, closed forms (q = 0 -> LSE = log n_keys,
uniform softmax), invariants (chunking / visiting-order invariance, permutation
round trips, RoPE relative-position property and norm preservation), and autograd of
an independently written dense formula.  The reference's own tests hold no golden
vectors for this path (tests/test_ring_attention.py uses unseeded randn and compares
with SDPA at run time, threshold 1e-4); the SDPA comparison is reproduced.  For the
Ulysses permutation and RoPE the reference has no test at all: those are pinned by the
brute-force / closed-form checks only (reference parity unpinned by reference tests).
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch

NEG_INF = float("-inf")


# --------------------------------------------------------------------------- positions
def ring_order(rank: int, world: int) -> List[int]:
    """KV chunk owner seen at step s by `rank`: (rank - s) mod W.
    ring_attention.py:39-40 (send right / receive from left), :110-115 (swap)."""
    return [(rank - s) % world for s in range(world)]


def contiguous_positions(rank: int, s_local: int) -> torch.Tensor:
    """Global token positions of cp-rank `rank`: data/dataloader.py:159-160."""
    return torch.arange(rank * s_local, (rank + 1) * s_local, dtype=torch.int64)


def zigzag_half_chunks(rank: int, world: int) -> Tuple[int, int]:
    """Load-balanced causal assignment (not in the reference): with 2W half-chunks,
    rank r holds half-chunk r and half-chunk 2W-1-r, in that local order."""
    return rank, 2 * world - 1 - rank


def zigzag_positions(rank: int, world: int, s_total: int) -> torch.Tensor:
    hc = s_total // (2 * world)
    a, b = zigzag_half_chunks(rank, world)
    return torch.cat([torch.arange(a * hc, (a + 1) * hc, dtype=torch.int64),
                      torch.arange(b * hc, (b + 1) * hc, dtype=torch.int64)])


def kv_head_of(q_head: int, n_rep: int) -> int:
    """repeat_kv repeats each kv head n_rep times consecutively (model/model.py:29-33),
    so q head h reads kv head h // n_rep."""
    return q_head // n_rep


# --------------------------------------------------------------------------- ring forward
def _expand_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    # [B, S, Hkv, D] -> [B, S, Hkv*n_rep, D]; index form of model/model.py:29-33
    if n_rep == 1:
        return x
    idx = torch.arange(x.shape[2] * n_rep) // n_rep
    return x[:, :, idx, :]


def ring_attention_recurrence(
    local_q: torch.Tensor,                      # [B, Sq, Hq, D]
    kv_chunks: Sequence[Tuple[torch.Tensor, torch.Tensor]],  # each [B, Sk, Hkv, D], visiting order
    q_pos: Optional[torch.Tensor] = None,       # [Sq] int64 global positions
    k_pos: Optional[Sequence[torch.Tensor]] = None,  # per chunk [Sk]
    causal: bool = False,
    compute_dtype: torch.dtype = torch.float32,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """The reference's online-softmax ring recurrence, one rank's share.

    Per chunk (ring_attention.py:66-107): S = (Q K^T) * scale; bm = max_k S;
    m' = max(m, bm); a = exp(m - m'); b = exp(bm - m'); P = exp(S - bm); bs = sum_k P;
    l = l*a + bs*b; O = O*a + (P V)*b; m = m'.  Finally O / l (:118).
    Returns (O [B,Sq,Hq,D], LSE [B,Hq,Sq]) with LSE = m + log l (implied, not in the
    reference).  Causal: key visible iff k_pos <= q_pos; a chunk with no visible key
    for any row is skipped; rows with no visible key in a visited chunk contribute
    nothing (the reference form would produce exp(-inf - -inf) = NaN there).
    """
    B, Sq, Hq, D = local_q.shape
    scale = 1.0 / math.sqrt(D)                                   # :20
    q_ = local_q.to(compute_dtype).transpose(1, 2)               # [B,H,Sq,D]  :66
    m = torch.full((B, Sq, Hq, 1), NEG_INF, dtype=compute_dtype)  # :26
    l = torch.zeros((B, Sq, Hq, 1), dtype=compute_dtype)          # :27
    o = torch.zeros((B, Sq, Hq, D), dtype=compute_dtype)          # :28
    for c, (k, v) in enumerate(kv_chunks):
        n_rep = Hq // k.shape[2]
        k_ = _expand_kv(k.to(compute_dtype), n_rep).transpose(1, 2)
        v_ = _expand_kv(v.to(compute_dtype), n_rep).transpose(1, 2)
        s = torch.matmul(q_, k_.transpose(-1, -2)) * scale        # :71
        s = s.transpose(1, 2)                                     # [B,Sq,H,Sk]  :76
        if causal:
            vis = k_pos[c][None, :] <= q_pos[:, None]             # [Sq,Sk]
            if not bool(vis.any()):
                continue
            s = s.masked_fill(~vis[None, :, None, :], NEG_INF)
        bm = torch.max(s, dim=-1, keepdim=True).values            # :79
        new_m = torch.maximum(m, bm)                              # :82
        safe_new = torch.where(torch.isinf(new_m), torch.zeros_like(new_m), new_m)
        safe_bm = torch.where(torch.isinf(bm), torch.zeros_like(bm), bm)
        a = torch.exp(m - safe_new)                               # :85
        b = torch.exp(bm - safe_new)                              # :86
        p = torch.exp(s - safe_bm)                                # :90
        bs = torch.sum(p, dim=-1, keepdim=True)                   # :94
        l = l * a + bs * b                                        # :95
        pv = torch.matmul(p.transpose(1, 2), v_).transpose(1, 2)  # :101-102
        o = o * a + pv * b                                        # :104
        m = new_m                                                 # :107
    safe_l = torch.where(l == 0, torch.ones_like(l), l)
    out = o / safe_l                                              # :118
    lse = (m + torch.log(l)).squeeze(-1).transpose(1, 2)          # [B,Hq,Sq]
    lse = torch.where(torch.isnan(lse), torch.full_like(lse, NEG_INF), lse)
    return out, lse


def merge_o_lse(o1, lse1, o2, lse2):
    """Pair-merge form of the same recurrence: two normalised partial results over
    disjoint key sets combine as LSE = logaddexp(lse1, lse2),
    O = O1*exp(lse1-LSE) + O2*exp(lse2-LSE).  o: [B,S,H,D]; lse: [B,H,S]."""
    lse = torch.logaddexp(lse1, lse2)
    safe = torch.where(torch.isinf(lse), torch.zeros_like(lse), lse)
    w1 = torch.exp(lse1 - safe).transpose(1, 2).unsqueeze(-1)
    w2 = torch.exp(lse2 - safe).transpose(1, 2).unsqueeze(-1)
    return o1 * w1 + o2 * w2, lse


# --------------------------------------------------------------------------- dense closed form
def dense_attention(q, k, v, q_pos=None, k_pos=None, causal=False, dtype=torch.float64):
    """softmax(Q K^T / sqrt(D) + mask) V and its log-sum-exp, written independently of
    the recurrence (one softmax over all keys).  q: [B,Sq,Hq,D]; k,v: [B,Sk,Hkv,D]."""
    B, Sq, Hq, D = q.shape
    n_rep = Hq // k.shape[2]
    qf = q.to(dtype).permute(0, 2, 1, 3)
    kf = k.to(dtype).repeat_interleave(n_rep, dim=2).permute(0, 2, 1, 3)
    vf = v.to(dtype).repeat_interleave(n_rep, dim=2).permute(0, 2, 1, 3)
    s = torch.einsum("bhqd,bhkd->bhqk", qf, kf) / math.sqrt(D)
    if causal:
        vis = k_pos[None, :] <= q_pos[:, None]
        s = s.masked_fill(~vis, NEG_INF)
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - torch.where(torch.isinf(lse), torch.zeros_like(lse), lse).unsqueeze(-1))
    o = torch.einsum("bhqk,bhkd->bhqd", p, vf).permute(0, 2, 1, 3)
    return o, lse


def dense_attention_grads(q, k, v, do, q_pos=None, k_pos=None, causal=False, dtype=torch.float64):
    """dQ, dK, dV of dense_attention by torch.autograd (GQA grads sum over the n_rep q
    heads of a group because repeat_interleave's backward sums)."""
    qd = q.detach().to(dtype).requires_grad_(True)
    kd = k.detach().to(dtype).requires_grad_(True)
    vd = v.detach().to(dtype).requires_grad_(True)
    o, lse = dense_attention(qd, kd, vd, q_pos, k_pos, causal, dtype)
    o.backward(do.to(dtype))
    return o.detach(), lse.detach(), qd.grad, kd.grad, vd.grad


def attention_backward_formula(q, k, v, o, lse, do, q_pos=None, k_pos=None, causal=False,
                               dtype=torch.float32):
    """The recompute backward the kernels implement, in dense form:
    D = rowsum(dO*O); P = exp(S*scale - LSE); dV = P^T dO; dP = dO V^T;
    dS = P*(dP - D); dQ = dS K * scale; dK = dS^T Q * scale.  Used by the CPU baseline
    (timed) and cross-checked against autograd in the tests."""
    B, Sq, Hq, D = q.shape
    Hkv = k.shape[2]
    n_rep = Hq // Hkv
    scale = 1.0 / math.sqrt(D)
    qf = q.to(dtype).permute(0, 2, 1, 3)
    kf = _expand_kv(k.to(dtype), n_rep).permute(0, 2, 1, 3)
    vf = _expand_kv(v.to(dtype), n_rep).permute(0, 2, 1, 3)
    dof = do.to(dtype).permute(0, 2, 1, 3)
    of = o.to(dtype).permute(0, 2, 1, 3)
    delta = (dof * of).sum(-1, keepdim=True)
    s = torch.matmul(qf, kf.transpose(-1, -2)) * scale
    if causal:
        vis = k_pos[None, :] <= q_pos[:, None]
        s = s.masked_fill(~vis, NEG_INF)
    safe = torch.where(torch.isinf(lse), torch.zeros_like(lse), lse).to(dtype)
    p = torch.exp(s - safe.unsqueeze(-1))
    dv = torch.matmul(p.transpose(-1, -2), dof)
    dp = torch.matmul(dof, vf.transpose(-1, -2))
    ds = p * (dp - delta)
    dq = torch.matmul(ds, kf) * scale
    dk = torch.matmul(ds.transpose(-1, -2), qf) * scale
    Sk = k.shape[1]
    dk = dk.reshape(B, Hkv, n_rep, Sk, D).sum(2).permute(0, 2, 1, 3)
    dv = dv.reshape(B, Hkv, n_rep, Sk, D).sum(2).permute(0, 2, 1, 3)
    return dq.permute(0, 2, 1, 3), dk, dv


# --------------------------------------------------------------------------- Ulysses permutation
def seq_all_to_all(shards: Sequence[torch.Tensor], scatter_dim: int, gather_dim: int) -> List[torch.Tensor]:
    """All ranks' outputs of SeqAllToAll.forward (parallel_cp.py:49-73) given all ranks'
    inputs: rank i receives, from every rank j in order, the i-th split of j's tensor
    along scatter_dim, and concatenates them along gather_dim."""
    W = len(shards)
    if W == 1:
        return [shards[0]]                                        # :55-56
    size = shards[0].size(scatter_dim)
    assert size % W == 0                                          # :61-63
    pieces = [list(torch.split(x.contiguous(), size // W, dim=scatter_dim)) for x in shards]  # :65
    return [torch.cat([pieces[j][i] for j in range(W)], dim=gather_dim) for i in range(W)]  # :71-73


# --------------------------------------------------------------------------- RoPE
def precompute_freqs_cis(dim: int, end: int, theta: float = 10000.0) -> torch.Tensor:
    """layers/layers.py:18-24: theta_i = theta^(-2i/dim), angle[t,i] = t*theta_i in fp32,
    result complex64 [end, dim/2]."""
    freqs = 1.0 / (theta ** (torch.arange(0, dim, 2)[: dim // 2].float() / dim))
    t = torch.arange(end)
    ang = torch.outer(t, freqs).float()
    return torch.complex(torch.cos(ang), torch.sin(ang))


def apply_rotary_emb(xq, xk, freqs_cis):
    """layers/layers.py:44-70: rotate adjacent pairs (x[2i], x[2i+1]) by angle[t,i] in
    fp32, cast back.  x: [B,S,H,D]; freqs_cis: [S, D/2] (shape must match, :34)."""
    def rot(x):
        assert freqs_cis.shape == (x.shape[1], x.shape[-1] // 2)
        xf = x.float().reshape(*x.shape[:-1], -1, 2)
        c = freqs_cis.real[None, :, None, :]
        s = freqs_cis.imag[None, :, None, :]
        re = xf[..., 0] * c - xf[..., 1] * s
        im = xf[..., 0] * s + xf[..., 1] * c
        return torch.stack([re, im], dim=-1).flatten(3).type_as(x)
    return rot(xq), rot(xk)


# --------------------------------------------------------------------------- work model
def n_pairs_causal(q_pos: torch.Tensor, k_pos: torch.Tensor) -> int:
    """Number of unmasked (query, key) pairs; positions sorted or not."""
    ks = torch.sort(k_pos).values
    return int(torch.searchsorted(ks, q_pos, right=True).sum())


# --------------------------------------------------------------------------- sampled checks at full size
def sampled_rows(q, k, v, q_pos, k_pos, causal, rows, do=None, dtype=torch.float64):
    """Dense closed form restricted to sampled query rows, for inputs too large for the dense oracle.
    q: [B,Sq,Hq,D]; k, v: [B,Sk,Hkv,D] (any row order; k_pos gives positions); rows: list of (b, h, i).
    Returns per row (o [D], lse, dq [D] or None).  Pinned against dense_attention_grads in the CPU tests."""
    D = q.shape[-1]
    n_rep = q.shape[2] // k.shape[2]
    scale = 1.0 / math.sqrt(D)
    out = []
    for (b, h, i) in rows:
        g = h // n_rep
        qi = q[b, i, h].to(dtype)
        kk, vv = k[b, :, g].to(dtype), v[b, :, g].to(dtype)
        s = (kk @ qi) * scale
        if causal:
            s = s.masked_fill(k_pos > q_pos[i], NEG_INF)
        lse = torch.logsumexp(s, 0)
        p = torch.exp(s - lse)
        o = p @ vv
        dq = None
        if do is not None:
            doi = do[b, i, h].to(dtype)
            dp = vv @ doi
            ds = p * (dp - (doi * o).sum())
            dq = (ds @ kk) * scale
        out.append((o, lse, dq))
    return out


def sampled_keys(q, k, v, o, lse, do, q_pos, k_pos, causal, keys, dtype=torch.float64):
    """dK and dV of sampled keys (b, g, j) from the recompute formula over ALL query rows and the
    n_rep query heads of the group, given the forward results o [B,Sq,Hq,D] and lse [B,Hq,Sq]."""
    D = q.shape[-1]
    n_rep = q.shape[2] // k.shape[2]
    scale = 1.0 / math.sqrt(D)
    out = []
    for (b, g, j) in keys:
        kj, vj = k[b, j, g].to(dtype), v[b, j, g].to(dtype)
        dk = torch.zeros(D, dtype=dtype)
        dv = torch.zeros(D, dtype=dtype)
        for h in range(g * n_rep, (g + 1) * n_rep):
            qq, dd, oo = q[b, :, h].to(dtype), do[b, :, h].to(dtype), o[b, :, h].to(dtype)
            s = (qq @ kj) * scale
            p = torch.exp(s - lse[b, h].to(dtype))
            if causal:
                p = torch.where(q_pos >= k_pos[j], p, torch.zeros_like(p))
            p = torch.where(torch.isfinite(p), p, torch.zeros_like(p))
            delta = (dd * oo).sum(-1)
            ds = p * (dd @ vj - delta)
            dk += (ds @ qq) * scale
            dv += p @ dd
        out.append((dk, dv))
    return out
