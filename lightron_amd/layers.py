"""RoPE helpers with the reference's conventions (layers/layers.py:18-70): input preparation
for the attention kernels, run with torch ops on whatever device the inputs live on."""
import torch


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


def apply_rotary_emb(xq, xk, freqs_cis):
    """Rotate adjacent pairs (x[2i], x[2i+1]) in fp32 and cast back (layers.py:44-70)."""
    xq_ = torch.view_as_complex(xq.float().reshape(*xq.shape[:-1], -1, 2))
    xk_ = torch.view_as_complex(xk.float().reshape(*xk.shape[:-1], -1, 2))
    fc = reshape_for_broadcast(freqs_cis, xq_)
    xq_out = torch.view_as_real(xq_ * fc).flatten(3)
    xk_out = torch.view_as_real(xk_ * fc).flatten(3)
    return xq_out.type_as(xq), xk_out.type_as(xk)
