"""RoPE with the reference's conventions (layers/layers.py:18-70).  The rotation is one streaming HIP kernel
(ltr_rope_apply) with the conjugate rotation as its gradient - or, for q, the prologue of the attention kernel itself
(block_attention(..., q_rope=rope_table(freqs_cis))); the angle table is built with torch ops exactly as the reference
builds it."""
import ctypes

import torch

from . import _lib


def precompute_freqs_cis(dim: int, end: int, theta: float = 10000.0, device=None) -> torch.Tensor:
    """complex64 [end, dim/2], angle[t, i] = t * theta^(-2i/dim) computed in fp32 (layers.py:18-24)."""
    freqs = 1.0 / (theta ** (torch.arange(0, dim, 2, device=device)[: dim // 2].float() / dim))
    t = torch.arange(end, device=device)
    freqs = torch.outer(t, freqs).float()
    return torch.polar(torch.ones_like(freqs), freqs)


def reshape_for_broadcast(freqs_cis: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    if freqs_cis.shape != (x.shape[1], x.shape[-1]):                     # layers.py:34
        raise AssertionError("freqs_cis shape %s does not match x shape %s"
                             % (tuple(freqs_cis.shape), (x.shape[1], x.shape[-1])))
    shape = [d if i == 1 or i == x.ndim - 1 else 1 for i, d in enumerate(x.shape)]
    return freqs_cis.view(*shape)


def _rope_launch(x: torch.Tensor, table: torch.Tensor, conj: bool) -> torch.Tensor:
    """x: [B, S, H, D] on the GPU (bf16 or fp32, last dim contiguous); table: fp32 [S, D/2, 2] (cos, sin)."""
    lib = _lib.load()
    B, S, H, D = x.shape
    if x.stride(-1) != 1:
        x = x.contiguous()
    out = torch.empty((B, S, H, D), dtype=x.dtype, device=x.device)
    a = _lib.RopeArgs()
    a.x, a.out, a.freqs = x.data_ptr(), out.data_ptr(), table.data_ptr()
    a.B, a.H, a.D, a.S = B, H, D, S
    for i in range(3):
        a.x_stride[i] = x.stride(i)
        a.out_stride[i] = out.stride(i)
    a.flags = 1 if conj else 0                                           # LTR_ROPE_CONJ
    a.io_dtype = _lib.LTR_BF16 if x.dtype == torch.bfloat16 else _lib.LTR_F32
    _lib.check(lib.ltr_rope_apply(ctypes.byref(a), torch.cuda.current_stream(x.device).cuda_stream), "ltr_rope_apply")
    return out


class _Rope(torch.autograd.Function):
    """x -> x * freqs_cis over adjacent pairs; the gradient is the rotation by the conjugate angles."""

    @staticmethod
    def forward(ctx, x, table):
        ctx.save_for_backward(table)
        return _rope_launch(x, table, False)

    @staticmethod
    def backward(ctx, grad):
        (table,) = ctx.saved_tensors
        return _rope_launch(grad, table, True), None


def rope_table(freqs_cis: torch.Tensor, device=None) -> torch.Tensor:
    """The complex64 table of precompute_freqs_cis as the fp32 [S, D/2, 2] (cos, sin) rows the HIP kernels read."""
    return torch.view_as_real(freqs_cis.to(device=device or freqs_cis.device, dtype=torch.complex64)).contiguous()


def rope_one(x: torch.Tensor, freqs_cis: torch.Tensor) -> torch.Tensor:
    """apply_rotary_emb for ONE GPU tensor (K, when q's rotation is fused into the attention kernel)."""
    return _rope_gpu(x, freqs_cis)


def _rope_gpu(x: torch.Tensor, freqs_cis: torch.Tensor) -> torch.Tensor:
    if x.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError("apply_rotary_emb on the GPU takes bf16 or fp32 tensors, got %s" % x.dtype)
    if x.shape[-1] % 8:
        raise ValueError("head dim must be a multiple of 8")
    if freqs_cis.shape != (x.shape[1], x.shape[-1] // 2):                # layers.py:34 (shape of the complex view)
        raise AssertionError("freqs_cis shape %s does not match x shape %s"
                             % (tuple(freqs_cis.shape), (x.shape[1], x.shape[-1] // 2)))
    table = torch.view_as_real(freqs_cis.to(device=x.device, dtype=torch.complex64)).contiguous()
    return _Rope.apply(x, table)


def apply_rotary_emb(xq, xk, freqs_cis):
    """Rotate adjacent pairs (x[2i], x[2i+1]) in fp32 and cast back (layers.py:44-70), on the GPU through the HIP
    kernel and only through it: tensors that live on the host are refused, like everywhere else in this package."""
    if not (xq.is_cuda and xk.is_cuda):
        raise RuntimeError("apply_rotary_emb takes GPU tensors (the HIP library has no CPU path)")
    return _rope_gpu(xq, freqs_cis), _rope_gpu(xk, freqs_cis)
