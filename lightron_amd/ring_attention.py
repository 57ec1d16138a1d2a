"""Drop-in for parallel/communication/ring_attention.py of the reference on ONE GPU.

`ring_attention_kernel(local_q, local_k, local_v, cp_group, tp_group)` keeps the reference's
five positional arguments and its [B, S_local, H, D] layout (ring_attention.py:10-19).  Where
the reference rotates K/V between ranks with batch_isend_irecv (:48-60, :110-115), here every
rank's KV chunk is already resident in HBM and `cp_group` is a `LocalRing` descriptor that
names them; the kernel visits them in the reference's order (rank r sees chunks r, r-1, ...
mod W).  A real torch.distributed ProcessGroup with more than one rank is refused: this
build has no collectives.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

from .attention import block_attention


class RingKVGrads:
    """fp32 dK / dV accumulators of a ring whose KV chunks live on this GPU, shared by the LocalRing descriptors of all
    its ranks: every rank's backward adds its contribution (the kernels accumulate in fp32), and finalize() makes the
    ONE cast to the chunks' dtype.  Without it autograd sums W bf16-rounded per-rank gradients.  In a real ring these
    are the accumulators that travel with the KV chunk."""

    def __init__(self, kv: Sequence):
        self.kv = list(kv)
        self.dk = [torch.zeros(k.shape, dtype=torch.float32, device=k.device) for k, _ in self.kv]
        self.dv = [torch.zeros(v.shape, dtype=torch.float32, device=v.device) for _, v in self.kv]

    def zero_(self):
        for t in self.dk + self.dv:
            t.zero_()

    def finalize(self, assign: bool = True):
        """[(dK, dV)] per rank in the chunks' dtype; with assign=True also added to k.grad / v.grad of leaf tensors."""
        from .attention import cast_to_bf16
        out = []
        for (k, v), dk, dv in zip(self.kv, self.dk, self.dv):
            gk = cast_to_bf16(dk) if k.dtype == torch.bfloat16 else dk.to(k.dtype)
            gv = cast_to_bf16(dv) if v.dtype == torch.bfloat16 else dv.to(v.dtype)
            if assign:
                for t, g in ((k, gk), (v, gv)):
                    if t.requires_grad and t.is_leaf:
                        t.grad = g.clone() if t.grad is None else t.grad + g
            out.append((gk, gv))
        return out


class LocalRing:
    """Stand-in for the cp ProcessGroup of a ring whose KV chunks all live on this GPU.

    rank, world_size : this rank's place in the ring.
    kv               : list of (k, v) per rank, in rank order, each [B, S_local, Hkv, D];
                       entry `rank` may be None (local_k / local_v are used).
    causal           : mask by global token position (the reference ring is non-causal).
    layout           : "contiguous" - rank r owns tokens [r*S_l, (r+1)*S_l)
                       (data/dataloader.py:159-160 of the reference);
                       "zigzag" - rank r owns half-chunks r and 2W-1-r of 2W, in that order.
    stepwise         : one kernel launch per ring step with the (O, LSE) merge fused in the
                       epilogue (the shape of a real ring, where chunks arrive one at a
                       time) instead of one launch that walks the whole chunk table.
    out_dtype        : dtype of the result (default: dtype of local_q).
    kv_grads         : a RingKVGrads over the same kv list, shared by all ranks' descriptors: the backward adds dK / dV
                       into its fp32 accumulators instead of returning per-rank gradients to autograd.
    """

    def __init__(self, rank: int, world_size: int, kv: Optional[Sequence] = None, causal: bool = False,
                 layout: str = "contiguous", stepwise: bool = False, out_dtype: Optional[torch.dtype] = None,
                 kv_grads: Optional[RingKVGrads] = None):
        if not (0 <= rank < world_size):
            raise ValueError("rank %d outside ring of %d" % (rank, world_size))
        if layout not in ("contiguous", "zigzag"):
            raise ValueError("unknown layout %r" % layout)
        self.rank, self.world_size = rank, world_size
        self.kv = list(kv) if kv is not None else [None] * world_size
        if len(self.kv) != world_size:
            raise ValueError("kv must have one entry per rank")
        self.causal, self.layout, self.stepwise, self.out_dtype = causal, layout, stepwise, out_dtype
        if kv_grads is not None and len(kv_grads.dk) != world_size:
            raise ValueError("kv_grads must cover one KV chunk per rank")
        self.kv_grads = kv_grads
        self.last_lse = None

    def order(self) -> List[int]:
        """Chunk owner visited at step s: (rank - s) mod W (ring_attention.py:39-40, 110-115)."""
        return [(self.rank - s) % self.world_size for s in range(self.world_size)]


def _chunk_table(ring: LocalRing, local_k, local_v, s_local: int):
    """KV chunks in visiting order with the global position of each chunk's first key."""
    W = ring.world_size
    ks, vs, pos = [], [], []
    dks, dvs = [], []
    acc = ring.kv_grads
    for j in ring.order():
        kv = ring.kv[j]
        if kv is None:
            if j != ring.rank:
                raise RuntimeError("LocalRing has no KV chunk for rank %d" % j)
            kv = (local_k, local_v)
        k, v = kv
        if ring.layout == "contiguous":
            ks.append(k)
            vs.append(v)
            pos.append(j * s_local)
            if acc is not None:
                dks.append(acc.dk[j])
                dvs.append(acc.dv[j])
        else:
            hc = s_local // 2
            ks += [k[:, :hc], k[:, hc:]]
            vs += [v[:, :hc], v[:, hc:]]
            pos += [j * hc, (2 * W - 1 - j) * hc]
            if acc is not None:
                dks += [acc.dk[j][:, :hc], acc.dk[j][:, hc:]]
                dvs += [acc.dv[j][:, :hc], acc.dv[j][:, hc:]]
    return ks, vs, pos, ((dks, dvs) if acc is not None else None)


def ring_attention_with_lse(local_q, local_k, local_v, cp_group) -> Tuple[torch.Tensor, torch.Tensor]:
    """Same computation, returning (O [B,S_local,H,D], LSE [B,H,S_local] fp32)."""
    if cp_group is None:
        ring = LocalRing(0, 1)
    elif isinstance(cp_group, LocalRing):
        ring = cp_group
    else:
        import torch.distributed as dist
        if dist.is_available() and dist.is_initialized() and dist.get_world_size(group=cp_group) == 1:
            ring = LocalRing(0, 1)
        else:
            raise NotImplementedError(
                "ring_attention_kernel: this build runs on one GPU and has no collectives; pass a LocalRing "
                "describing the KV chunks resident in HBM instead of a multi-rank ProcessGroup")
    S_local = local_q.shape[1]
    W = ring.world_size
    if ring.layout == "zigzag":
        if S_local % 2:
            raise ValueError("zigzag layout needs an even local sequence length")
        hc = S_local // 2
        q_pos0, q_split = (ring.rank * hc, (2 * W - 1 - ring.rank) * hc), hc
    else:
        q_pos0, q_split = (ring.rank * S_local, ring.rank * S_local), S_local
    ks, vs, pos, grad_acc = _chunk_table(ring, local_k, local_v, S_local)
    if grad_acc is not None and ring.kv[ring.rank] is None:
        raise RuntimeError("kv_grads needs the ring's own chunk in LocalRing.kv (entry %d is None)" % ring.rank)
    # a ring step delivers one rank's chunk: one table entry, or the two half-chunks of a zig-zag chunk in ONE launch (the
    # dK/dV and forward kernels then see twice the keys per launch: a block for every CU where a half-chunk leaves half idle)
    step = (2 if ring.layout == "zigzag" else 1) if ring.stepwise else False
    o, lse = block_attention(local_q, ks, vs, pos, q_pos0, q_split, ring.causal, None, step,
                             ring.out_dtype, grad_acc)
    return o, lse


def ring_attention_kernel(local_q, local_k, local_v, cp_group, tp_group=None):
    """local_q/k/v: [B, S_local, H_local, D] -> O [B, S_local, H_local, D]
    (ring_attention.py:10-13, :119).  tp_group is accepted and unused, as in the reference."""
    o, lse = ring_attention_with_lse(local_q, local_k, local_v, cp_group)
    if isinstance(cp_group, LocalRing):
        cp_group.last_lse = lse
    return o
