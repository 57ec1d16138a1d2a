"""The reference's non-CP attention layer (model/model.py:11-34, 123-202) on the HIP kernels: same constructor
arguments, parameter names (wq, wk, wv, wo) and forward(x, freqs_cis) -> [B, S, dim] contract, so a
TransformerBlock-shaped caller (model/model.py:228-229) or ContextParallelAttention can hold it unchanged.
Differences, on purpose: K and V keep their n_kv_heads heads all the way into the kernel (kv head = q head //
n_rep, the mapping of repeat_kv, model/model.py:11-34) instead of being materialised n_rep times, and they are
viewed with n_kv_heads (the reference views them with n_heads, model/model.py:165-167, which only works for
n_kv_heads == n_heads); tensor parallel linears are out of scope (tp_size must be 1)."""
import torch
from torch import nn

from .attention import block_attention
from .layers import apply_rotary_emb, rope_one, rope_table


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[B, S, Hkv, D] -> [B, S, Hkv * n_rep, D], every kv head repeated n_rep times consecutively
    (model/model.py:11-34).  Kept for callers of the reference's helper; Attention does not need it."""
    if n_rep == 1:
        return x
    B, S, Hkv, D = x.shape
    return x[:, :, :, None, :].expand(B, S, Hkv, n_rep, D).reshape(B, S, Hkv * n_rep, D)


class Attention(nn.Module):
    def __init__(self, args):
        super().__init__()
        self.tp_size = getattr(args, "tp_size", 1)
        if self.tp_size != 1:
            raise NotImplementedError("lightron_amd.Attention runs on one GPU: tp_size must be 1")
        self.n_heads = args.n_heads
        n_kv = getattr(args, "n_kv_heads", None)
        self.n_kv_heads = args.n_heads if n_kv is None else n_kv
        if self.n_heads % self.n_kv_heads:
            raise ValueError("n_heads must be a multiple of n_kv_heads")
        self.head_dim = args.dim // args.n_heads
        self.n_rep = self.n_heads // self.n_kv_heads
        self.wq = nn.Linear(args.dim, self.n_heads * self.head_dim, bias=False)
        self.wk = nn.Linear(args.dim, self.n_kv_heads * self.head_dim, bias=False)
        self.wv = nn.Linear(args.dim, self.n_kv_heads * self.head_dim, bias=False)
        self.wo = nn.Linear(self.n_heads * self.head_dim, args.dim, bias=False)

    def forward(self, x, freqs_cis):
        B, S, _ = x.shape
        xq = self.wq(x).view(B, S, self.n_heads, self.head_dim)
        xk = self.wk(x).view(B, S, self.n_kv_heads, self.head_dim)
        xv = self.wv(x).view(B, S, self.n_kv_heads, self.head_dim)
        # RoPE (model.py:183, before any head repetition): K in one streaming pass; q inside the attention kernel, whose
        # prologue rotates each row in registers (and whose dQ epilogue rotates the gradient back) when q is bf16
        # causal attention, scale 1/sqrt(D), [B, S, H, D] in and out: no transposes, no repeat_kv copy
        if xq.dtype == torch.bfloat16:
            if freqs_cis.shape != (S, self.head_dim // 2):               # layers.py:34
                raise AssertionError("freqs_cis shape %s does not match x shape %s" % (tuple(freqs_cis.shape), (S, self.head_dim // 2)))
            xk = rope_one(xk, freqs_cis)
            out, _ = block_attention(xq, [xk], [xv], [0], 0, None, causal=True, q_rope=rope_table(freqs_cis, xq.device))
        else:
            xq, xk = apply_rotary_emb(xq, xk, freqs_cis)
            out, _ = block_attention(xq, [xk], [xv], [0], 0, None, causal=True)
        return self.wo(out.reshape(B, S, -1))
