"""Drop-in for parallel/parallel_cp.py of the reference (Ulysses-style context parallelism)
on ONE GPU.

The reference exchanges sequence shards for head shards with dist.all_to_all
(parallel_cp.py:49-73).  Here one process stands in for all W ranks of the cp group: a
tensor that passes through `SeqAllToAll` carries a leading rank dimension of size W
(``x[r]`` is what rank r would hold) and the exchange is an index permutation on the device.
`scatter_dim` / `gather_dim` keep their per-rank meaning (they index ``x[r]``).  With
group=None or a one-rank group the op is the identity, as in the reference (:55-56, :82-83).
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .attention import block_attention
from .layers import rope_one, rope_table


class LocalCPGroup:
    """Stand-in for the cp ProcessGroup: `world_size` ranks emulated by one process."""

    def __init__(self, world_size: int):
        if world_size < 1:
            raise ValueError("world_size must be >= 1")
        self.world_size = world_size

    def size(self) -> int:
        return self.world_size


def _world_size(group) -> int:
    if group is None:
        return 1
    if isinstance(group, LocalCPGroup):
        return group.world_size
    import torch.distributed as dist
    if dist.is_available() and dist.is_initialized() and dist.get_world_size(group) == 1:
        return 1
    raise NotImplementedError("SeqAllToAll: this build runs on one GPU and has no collectives; pass a "
                              "LocalCPGroup (rank-stacked tensors) instead of a multi-rank ProcessGroup")


def _exchange(x: torch.Tensor, scatter_dim: int, gather_dim: int, W: int) -> torch.Tensor:
    """x: [W_src, *shard].  out[i] = cat_j(split(x[j], scatter_dim)[i], gather_dim)
    (parallel_cp.py:65-73 for every rank i at once)."""
    if x.shape[0] != W:
        raise RuntimeError("rank-stacked tensor must have leading dim %d, got %s" % (W, tuple(x.shape)))
    nd = x.dim() - 1
    sd, gd = scatter_dim % nd, gather_dim % nd
    size = x.size(sd + 1)
    assert size % W == 0, f"Input dim {scatter_dim} size {size} not divisible by CP size {W}"   # :61-63
    y = x.unflatten(sd + 1, (W, size // W))      # [W_src, ..., W_dst, chunk, ...]
    y = y.movedim(sd + 1, 0)                     # [W_dst, W_src, *shard with chunk at sd]
    y = y.movedim(1, gd + 1)                     # W_src just before the gather dim
    return y.flatten(gd + 1, gd + 2).contiguous()


class SeqAllToAll(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input_tensor, scatter_dim, gather_dim, group):
        ctx.scatter_dim, ctx.gather_dim, ctx.group = scatter_dim, gather_dim, group
        W = _world_size(group)
        if W == 1:
            return input_tensor
        return _exchange(input_tensor, scatter_dim, gather_dim, W)

    @staticmethod
    def backward(ctx, grad_output):
        # forward: scatter(dim1) -> exchange -> gather(dim2); backward swaps the dims (:75-96)
        W = _world_size(ctx.group)
        if W == 1:
            return grad_output, None, None, None
        return _exchange(grad_output, ctx.gather_dim, ctx.scatter_dim, W), None, None, None


def _all_to_all(input_, scatter_dim, gather_dim, group):
    return SeqAllToAll.apply(input_, scatter_dim, gather_dim, group)


class ContextParallelAttention(nn.Module):
    """Wrapper with the reference's constructor and forward (parallel_cp.py:120-245).

    `local_attn_module` supplies wq / wk / wv / wo and n_heads; `args` supplies n_heads, dim
    and tp_size.  The reference finds its cp group in a global device mesh; here it is passed
    as `cp_group` (a LocalCPGroup).  Without one the wrapped module is called unchanged
    (:161-162).  With one, `x` is rank-stacked [W, B, S_local, Hidden] and so is the result.

    literal=True follows the reference step by step (three seq->head exchanges, RoPE on the
    global sequence, causal attention on [B, S, H/W, D], head->seq exchange).  The default
    path gives the same result without moving data: each rank's sequence shard is one KV
    chunk of the kernel's chunk table, all heads are processed in one launch per Q shard, and
    the two exchanges cancel.
    """

    def __init__(self, local_attn_module, args, cp_group=None, literal: bool = False, causal: bool = True):
        super().__init__()
        self.local_attn = local_attn_module
        self.num_heads = args.n_heads
        if hasattr(local_attn_module, "n_heads"):
            self.num_heads = local_attn_module.n_heads
        else:
            self.num_heads = args.n_heads // getattr(args, "tp_size", 1)
        self.num_kv_heads = getattr(local_attn_module, "n_kv_heads", None) or self.num_heads
        self.head_dim = args.dim // args.n_heads
        self.cp_group = cp_group
        self.literal, self.causal = literal, causal
        if cp_group is not None:
            W = _world_size(cp_group)
            assert self.num_heads % W == 0, \
                f"Context Parallelism requires local_num_heads ({self.num_heads}) to be divisible by cp_size ({W})."

    def forward(self, x, freqs_cis):
        if self.cp_group is None:
            return self.local_attn(x, freqs_cis)
        W = _world_size(self.cp_group)
        if x.dim() != 4 or x.shape[0] != W:
            raise RuntimeError("with a LocalCPGroup x must be rank-stacked [W, B, S_local, Hidden]")
        _, B, S_local, _ = x.shape
        S_global = S_local * W
        assert freqs_cis.shape[0] >= S_global, f"freqs_cis too short: {freqs_cis.shape[0]} < S_global {S_global}"
        H, Hkv, D = self.num_heads, self.num_kv_heads, self.head_dim
        xq = self.local_attn.wq(x).view(W, B, S_local, H, D)
        xk = self.local_attn.wk(x).view(W, B, S_local, Hkv, D)
        xv = self.local_attn.wv(x).view(W, B, S_local, Hkv, D)
        fc = freqs_cis[:S_global]
        if self.literal:
            if Hkv % W:
                raise RuntimeError("literal Ulysses path needs n_kv_heads divisible by the cp size")
            xq = _all_to_all(xq, 2, 1, self.cp_group)            # [W, B, S_global, H/W, D]
            xk = _all_to_all(xk, 2, 1, self.cp_group)
            xv = _all_to_all(xv, 2, 1, self.cp_group)
            qf, kf, vf = (t.reshape(W * B, S_global, -1, D) for t in (xq, xk, xv))
            qf, kf = rope_one(qf, fc), rope_one(kf, fc)          # one streaming pass per tensor (q and k may differ in heads)
            o, _ = block_attention(qf, [kf], [vf], [0], 0, None, self.causal)
            o = o.view(W, B, S_global, H // W, D)
            o = _all_to_all(o, 1, 2, self.cp_group)              # [W, B, S_local, H, D]
        else:
            # RoPE at global positions (:215-219): every K shard is rotated once, in one streaming pass (it is read by
            # every later q shard); q is rotated inside the attention kernel's prologue, dQ rotated back in the dQ
            # kernel's epilogue (bf16; fp32 inputs take the streaming pass for q as well)
            outs = []
            fused = xq.dtype == torch.bfloat16
            table = rope_table(fc, xq.device) if fused else None
            qs, ks = [], []
            for j in range(W):
                fj = fc[j * S_local:(j + 1) * S_local]
                ks.append(rope_one(xk[j], fj))
                qs.append(xq[j] if fused else rope_one(xq[j], fj))
            vs = [xv[j] for j in range(W)]
            pos = [j * S_local for j in range(W)]
            for j in range(W):
                n = j + 1 if self.causal else W                  # later shards are fully masked
                oj, _ = block_attention(qs[j], ks[:n], vs[:n], pos[:n], j * S_local, None, self.causal, q_rope=table)
                outs.append(oj)
            o = torch.stack(outs, 0)
        return self.local_attn.wo(o.flatten(3))

