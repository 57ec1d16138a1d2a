"""Host side of the block-attention C ABI: argument marshalling and the autograd Function.

Tensors are logical [B, S, H, D] with arbitrary batch/seq/head strides and a contiguous
last dim, so [B,H,S,D] storage (pass ``x.transpose(1, 2)``) and head-slice views work
without copies.  All compute happens in the HIP library; there is no PyTorch fallback.
"""
from __future__ import annotations

import ctypes
import math
import os
import threading
from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib

_DT = {torch.bfloat16: _lib.LTR_BF16, torch.float32: _lib.LTR_F32}


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_ptr(dev) -> int:
    """hipStream_t of torch's current stream on `dev`, as an integer."""
    if _raw_stream is not None:
        return _raw_stream(dev.index if dev.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(dev).cuda_stream


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on_device(dev):
    """Context in which `dev` is the current device: the library launches on the CURRENT device.  The common case (it
    already is) costs one query instead of a device switch and back."""
    if dev.index is None or dev.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(dev)


def _s3(t: torch.Tensor):
    return (ctypes.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))


def _req(t: torch.Tensor, name: str):
    if not t.is_cuda:
        raise RuntimeError("%s must be a GPU tensor (the HIP library has no CPU path)" % name)
    if t.dim() != 4 or (t.numel() > 0 and t.stride(3) != 1):
        raise RuntimeError("%s must be [B,S,H,D] with a contiguous last dim, got shape %s strides %s"
                           % (name, tuple(t.shape), t.stride()))


def _same_strides(ts: Sequence[torch.Tensor]) -> bool:
    s0 = ts[0].stride()
    return all(t.stride() == s0 for t in ts)


_warned_repack = False


def _common_layout(ts):
    """The ABI carries ONE stride triple for all K chunks (and one for all V chunks).  Chunks that already share it -
    slices of one tensor along the sequence, or separate tensors of equal shape - pass through untouched.  Chunks whose
    strides differ (separate tensors of unequal length have different batch strides) take the SLOW PATH: they are
    copied into one [B, sum S, H, D] buffer (torch.cat: a pass over every chunk, in the forward and again in the
    backward) and returned as its sequence slices.  Warns once per process; callers on a hot path should hand in slices
    of one buffer."""
    if len(ts) == 1 or _same_strides(ts):
        return list(ts)
    global _warned_repack
    if not _warned_repack:
        _warned_repack = True
        import warnings
        warnings.warn("lightron_amd: KV chunks with different strides are packed into one buffer on every call "
                      "(a copy of every chunk); pass sequence slices of one tensor to avoid it", stacklevel=3)
    buf = torch.cat([t for t in ts], dim=1)
    out, start = [], 0
    for t in ts:
        out.append(buf[:, start:start + t.shape[1]])
        start += t.shape[1]
    return out


def _norm_chunks(ks, vs):
    """The ABI carries one stride triple for all K chunks and one for all V chunks."""
    return _common_layout(ks), _common_layout(vs)


def _rope_table_check(t, D, device):
    if (t.dtype != torch.float32 or t.dim() != 3 or t.shape[1] != D // 2 or t.shape[2] != 2 or not t.is_contiguous()
            or t.device != device):
        raise RuntimeError("the RoPE table must be a contiguous fp32 [n_pos, D/2, 2] (cos, sin) tensor on q's device")


def _qpos(q_pos0, Sq, q_split):
    if isinstance(q_pos0, int):
        q_pos0 = (q_pos0, q_pos0)
    if q_split is None:
        q_split = Sq
    return (ctypes.c_int64 * 2)(int(q_pos0[0]), int(q_pos0[1])), int(q_split)


def attn_fwd(q: torch.Tensor, ks: Sequence[torch.Tensor], vs: Sequence[torch.Tensor], k_pos0: Sequence[int],
             q_pos0=0, q_split: Optional[int] = None, causal: bool = False, scale: Optional[float] = None,
             out: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None, merge: bool = False,
             out_dtype: Optional[torch.dtype] = None, q_rope: Optional[torch.Tensor] = None,
             q_rot_out: Optional[torch.Tensor] = None, fwd_rows: Optional[int] = None,
             f32_scalar: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """One Q chunk against a table of KV chunks -> (O [B,Sq,Hq,D], LSE [B,Hq,Sq] fp32).
    With merge=True, `out`/`lse` hold an earlier partial result which is merged in place.
    q_rope: fp32 [n_pos, D/2, 2] (cos, sin) table whose row p belongs to global position p: q is un-rotated and the
    kernel's prologue applies RoPE to it (LTR_ROPE_Q; bf16 only); q_rot_out (bf16, like q) receives the rotated q.
    fwd_rows: None (the library chooses), 256 or 512 query rows per block (512: bf16 with head dim 64 only).
    f32_scalar: fp32 inputs only - the scalar fp32 kernel instead of the matrix-pipe one (LTR_FWD_F32_SCALAR)."""
    lib = _lib.load()
    _req(q, "q")
    B, Sq, Hq, D = q.shape
    ks, vs = _norm_chunks(ks, vs)
    for k, v in zip(ks, vs):
        _req(k, "k")
        _req(v, "v")
        if k.dtype != q.dtype or v.dtype != q.dtype or k.shape != v.shape or k.shape[0] != B or k.shape[3] != D:
            raise RuntimeError("k/v chunk shape or dtype mismatch")
    Hkv = ks[0].shape[2]
    if q.dtype not in _DT:
        raise RuntimeError("unsupported dtype %s" % q.dtype)
    if out is None:
        if merge:
            raise RuntimeError("merge=True needs the earlier partial result in out/lse")
        out = torch.empty((B, Sq, Hq, D), dtype=out_dtype or q.dtype, device=q.device)
        lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=q.device)
    _req(out, "out")
    if lse is None or lse.dtype != torch.float32 or not lse.is_contiguous() or tuple(lse.shape) != (B, Hq, Sq):
        raise RuntimeError("lse must be a contiguous fp32 [B,Hq,Sq] tensor")
    if q.numel() == 0:          # no query rows: the reference's matmuls return an empty result as well
        return out, lse
    a = _lib.FwdArgs()
    a.q, a.o, a.lse = q.data_ptr(), out.data_ptr(), lse.data_ptr()
    a.B, a.Hq, a.Hkv, a.D, a.Sq = B, Hq, Hkv, D, Sq
    a.q_stride, a.o_stride = _s3(q), _s3(out)
    a.k_stride, a.v_stride = _s3(ks[0]), _s3(vs[0])
    a.q_pos0, a.q_split = _qpos(q_pos0, Sq, q_split)
    a.scale = float(scale if scale is not None else 1.0 / math.sqrt(D))
    a.io_dtype, a.o_dtype = _DT[q.dtype], _DT[out.dtype]
    rope_flag = _lib.LTR_FWD_F32_SCALAR if f32_scalar else 0
    if fwd_rows is not None:
        if fwd_rows not in (256, 512):
            raise RuntimeError("fwd_rows must be None, 256 or 512")
        rope_flag |= _lib.LTR_FWD_ROWS_256 if fwd_rows == 256 else _lib.LTR_FWD_ROWS_512
    if q_rope is not None:
        _rope_table_check(q_rope, D, q.device)
        a.rope_freqs, a.rope_pos0, a.rope_len = q_rope.data_ptr(), 0, q_rope.shape[0]
        rope_flag |= _lib.LTR_ROPE_Q
        if q_rot_out is not None:
            _req(q_rot_out, "q_rot_out")
            if q_rot_out.dtype != torch.bfloat16 or q_rot_out.shape != q.shape:
                raise RuntimeError("q_rot_out must be a bf16 tensor shaped like q")
            a.q_rot, a.q_rot_stride = q_rot_out.data_ptr(), _s3(q_rot_out)
    elif q_rot_out is not None:
        raise RuntimeError("q_rot_out needs q_rope")
    stream = _stream_ptr(q.device)
    n = len(ks)
    with _on_device(q.device):
        for start in range(0, n, _lib.LTR_MAX_CHUNKS):
            stop = min(n, start + _lib.LTR_MAX_CHUNKS)
            a.n_chunks = stop - start
            for i in range(start, stop):
                ch = a.chunk[i - start]
                ch.k, ch.v, ch.dk, ch.dv = ks[i].data_ptr(), vs[i].data_ptr(), None, None
                ch.sk, ch.pos0 = ks[i].shape[1], int(k_pos0[i])
            a.flags = (_lib.LTR_CAUSAL if causal else 0) | (_lib.LTR_MERGE if (merge or start > 0) else 0) | rope_flag
            _lib.check(lib.ltr_attn_fwd(ctypes.byref(a), stream), "ltr_attn_fwd")
    return out, lse


def attn_delta(o: torch.Tensor, do: torch.Tensor) -> torch.Tensor:
    lib = _lib.load()
    _req(o, "o")
    _req(do, "dO")
    B, Sq, Hq, D = o.shape
    delta = torch.empty((B, Hq, Sq), dtype=torch.float32, device=o.device)
    if o.numel() == 0:
        return delta
    a = _lib.DeltaArgs()
    a.o, a.d_o, a.delta = o.data_ptr(), do.data_ptr(), delta.data_ptr()
    a.B, a.Hq, a.D, a.Sq = B, Hq, D, Sq
    a.o_stride, a.do_stride = _s3(o), _s3(do)
    a.o_dtype, a.do_dtype = _DT[o.dtype], _DT[do.dtype]
    with _on_device(o.device):
        _lib.check(lib.ltr_attn_bwd_delta(ctypes.byref(a), _stream_ptr(o.device)), "ltr_attn_bwd_delta")
    return delta


def attn_bwd_accumulate(q, do, lse, delta, ks, vs, k_pos0, dq_acc, dk_accs, dv_accs, q_pos0=0, q_split=None,
                        causal=False, scale=None, do_dq=True, do_dkdv=True, o=None, library_scratch=False, dq_rope=None,
                        dkdv_keys=None, dq_rows=None, f32_scalar=False):
    """Adds this Q chunk's contribution into the fp32 accumulators dq_acc / dk_accs / dv_accs.
    do_dq / do_dkdv select which of the two backward kernels are enqueued.  dq_acc may instead be a bf16
    tensor: it then RECEIVES dQ (LTR_DQ_BF16), which is only right when ks / vs hold every KV chunk these
    queries can see and fit one launch (at most 32 chunks).  With o (the bf16 forward output) given, delta is a
    workspace: the dQ kernel of the first launch computes rowsum(dO * O) into it (LTR_DELTA_FROM_O) and no
    attn_delta call is needed; this needs do_dq.  dk_accs / dv_accs may be bf16 tensors as well: they then RECEIVE
    dK / dV (LTR_DKDV_BF16; every key is written), which is only right when q holds every query row that sees
    these keys - one rank's own backward, not a ring step whose dK/dV are summed over ranks.
    library_scratch=True calls ltr_attn_bwd_noalloc instead: delta is ignored (pass None), DELTA lives in the library's
    fixed scratch array (at most LTR_NOALLOC_MAX_ROWS = B*Hq*Sq rows; calls that overlap on one GPU race on it), o is
    required and the library allocates nothing.
    dq_rope: the (cos, sin) table of attn_fwd's q_rope; q is then the ROTATED q (q_rot_out of that forward) and the dQ
    kernel's epilogue rotates dQ back by the conjugate angles (LTR_ROPE_DQ): dq is the gradient of the un-rotated q.
    dkdv_keys: None (the library chooses), 128 or 256 keys per block of the dK/dV kernel (256: bf16 with head dim 64 only).
    dq_rows: None, 256 or 512 query rows per block of the dQ kernel (512: bf16 with head dim 64 only).
    f32_scalar: fp32 inputs only - the scalar fp32 kernels instead of the matrix-pipe ones (LTR_BWD_F32_SCALAR)."""
    lib = _lib.load()
    if library_scratch and (o is None or not do_dq):
        raise RuntimeError("library_scratch needs o (DELTA is computed from it) and do_dq")
    _req(q, "q")
    _req(do, "dO")
    B, Sq, Hq, D = q.shape
    ks, vs = _norm_chunks(ks, vs)
    if not (_same_strides(dk_accs) and _same_strides(dv_accs)):
        raise RuntimeError("dk/dv accumulators must share one stride triple each")
    dq_direct = dq_acc.dtype == torch.bfloat16
    if dq_direct and do_dq and len(ks) > _lib.LTR_MAX_CHUNKS:
        raise RuntimeError("a bf16 dQ output needs all KV chunks in one launch (at most %d)" % _lib.LTR_MAX_CHUNKS)
    dkdv_direct = dk_accs[0].dtype == torch.bfloat16
    for t in list(dk_accs) + list(dv_accs):
        if t.dtype != dk_accs[0].dtype:
            raise RuntimeError("dK / dV tensors must share one dtype (fp32 accumulators or bf16 results)")
    for t in ([] if dq_direct else [dq_acc]) + ([] if dkdv_direct else list(dk_accs) + list(dv_accs)):
        _req(t, "accumulator")
        if t.dtype != torch.float32:
            raise RuntimeError("gradient accumulators must be fp32")
    if dq_direct:
        _req(dq_acc, "dQ")
    if dkdv_direct:
        for t in list(dk_accs) + list(dv_accs):
            _req(t, "dK / dV")
    if q.numel() == 0:          # no query rows: nothing to add; results that this call was to write are zero
        if dkdv_direct and do_dkdv:
            for t in list(dk_accs) + list(dv_accs):
                t.zero_()
        return
    a = _lib.BwdArgs()
    a.q, a.d_o, a.lse, a.dq = q.data_ptr(), do.data_ptr(), lse.data_ptr(), dq_acc.data_ptr()
    a.delta = None if library_scratch else delta.data_ptr()
    a.B, a.Hq, a.Hkv, a.D, a.Sq = B, Hq, ks[0].shape[2], D, Sq
    a.q_stride, a.do_stride, a.dq_stride = _s3(q), _s3(do), _s3(dq_acc)
    a.k_stride, a.v_stride = _s3(ks[0]), _s3(vs[0])
    a.dk_stride, a.dv_stride = _s3(dk_accs[0]), _s3(dv_accs[0])
    a.q_pos0, a.q_split = _qpos(q_pos0, Sq, q_split)
    a.scale = float(scale if scale is not None else 1.0 / math.sqrt(D))
    a.flags = ((_lib.LTR_CAUSAL if causal else 0) | (0 if do_dq else _lib.LTR_NO_DQ)
               | (0 if do_dkdv else _lib.LTR_NO_DKDV) | (_lib.LTR_DQ_BF16 if dq_direct else 0)
               | (_lib.LTR_DKDV_BF16 if dkdv_direct else 0) | (_lib.LTR_BWD_F32_SCALAR if f32_scalar else 0))
    a.io_dtype = _DT[q.dtype]
    if dkdv_keys is not None:
        if dkdv_keys not in (128, 256):
            raise RuntimeError("dkdv_keys must be None, 128 or 256")
        a.flags |= _lib.LTR_DKDV_KEYS_128 if dkdv_keys == 128 else _lib.LTR_DKDV_KEYS_256
    if dq_rows is not None:
        if dq_rows not in (256, 512):
            raise RuntimeError("dq_rows must be None, 256 or 512")
        a.flags |= _lib.LTR_DQ_ROWS_256 if dq_rows == 256 else _lib.LTR_DQ_ROWS_512
    if dq_rope is not None:
        _rope_table_check(dq_rope, D, q.device)
        if not do_dq:
            raise RuntimeError("dq_rope rotates dQ in the dQ kernel's epilogue: do_dq must be set")
        a.rope_freqs, a.rope_pos0, a.rope_len = dq_rope.data_ptr(), 0, dq_rope.shape[0]
        a.flags |= _lib.LTR_ROPE_DQ
    if o is not None:
        if not do_dq:
            raise RuntimeError("delta from o is computed by the dQ kernel: do_dq must be set")
        if o.dtype != torch.bfloat16:
            raise RuntimeError("delta from o needs the bf16 forward output")
        _req(o, "o")
        a.o, a.o_stride = o.data_ptr(), _s3(o)
    base_flags = a.flags
    stream = _stream_ptr(q.device)
    n = len(ks)
    with _on_device(q.device):
        for start in range(0, n, _lib.LTR_MAX_CHUNKS):
            stop = min(n, start + _lib.LTR_MAX_CHUNKS)
            a.n_chunks = stop - start
            a.flags = base_flags | (_lib.LTR_DELTA_FROM_O if (o is not None and start == 0) else 0)
            for i in range(start, stop):
                ch = a.chunk[i - start]
                ch.k, ch.v = ks[i].data_ptr(), vs[i].data_ptr()
                ch.dk, ch.dv = dk_accs[i].data_ptr(), dv_accs[i].data_ptr()
                ch.sk, ch.pos0 = ks[i].shape[1], int(k_pos0[i])
            if library_scratch:
                _lib.check(lib.ltr_attn_bwd_noalloc(ctypes.byref(a), stream), "ltr_attn_bwd_noalloc")
            else:
                _lib.check(lib.ltr_attn_bwd(ctypes.byref(a), stream), "ltr_attn_bwd")


def attn_plan(B: int, Hq: int, Hkv: int, D: int, Sq: int, chunk_lens: Sequence[int], k_pos0: Sequence[int], q_pos0=0,
              q_split: Optional[int] = None, causal: bool = False, dtype: torch.dtype = torch.bfloat16, fwd_rows=None,
              dq_rows=None, dkdv_keys=None, f32_scalar: bool = False) -> dict:
    """Which kernels the library would launch for this problem on the current device (ltr_attn_plan: a host call, no
    tensors needed; at most 32 chunks = one launch): block sizes, block counts and the kernels' names as a profiler
    shows them.  fwd_rows / dq_rows / dkdv_keys force a size like the arguments of attn_fwd / attn_bwd_accumulate."""
    lib = _lib.load()
    a = _lib.BwdArgs()
    a.B, a.Hq, a.Hkv, a.D, a.Sq, a.n_chunks = B, Hq, Hkv, D, Sq, len(chunk_lens)
    a.q_pos0, a.q_split = _qpos(q_pos0, Sq, q_split)
    a.io_dtype = _DT[dtype]
    a.flags = (_lib.LTR_CAUSAL if causal else 0) | ((_lib.LTR_FWD_F32_SCALAR | _lib.LTR_BWD_F32_SCALAR) if f32_scalar else 0)
    for val, lo, hi, name in ((fwd_rows, _lib.LTR_FWD_ROWS_256, _lib.LTR_FWD_ROWS_512, "fwd_rows"),
                              (dq_rows, _lib.LTR_DQ_ROWS_256, _lib.LTR_DQ_ROWS_512, "dq_rows"),
                              (dkdv_keys, _lib.LTR_DKDV_KEYS_128, _lib.LTR_DKDV_KEYS_256, "dkdv_keys")):
        if val is not None:
            sizes = (128, 256) if name == "dkdv_keys" else (256, 512)
            if val not in sizes:
                raise RuntimeError("%s must be None, %d or %d" % ((name,) + sizes))
            a.flags |= lo if val == sizes[0] else hi
    for i, (sk, p0) in enumerate(zip(chunk_lens, k_pos0)):
        a.chunk[i].sk, a.chunk[i].pos0 = int(sk), int(p0)
    out = _lib.AttnPlan()
    _lib.check(lib.ltr_attn_plan(ctypes.byref(a), ctypes.byref(out)), "ltr_attn_plan")
    return {"compute_units": out.compute_units,
            "fwd": {"kernel": out.fwd_kernel.decode(), "rows": out.fwd_rows, "paired": bool(out.fwd_paired), "blocks": out.fwd_blocks},
            "dq": {"kernel": out.dq_kernel.decode(), "rows": out.dq_rows, "paired": bool(out.dq_paired), "blocks": out.dq_blocks},
            "dkdv": {"kernel": out.dkdv_kernel.decode(), "keys": out.dkdv_keys, "blocks": out.dkdv_blocks}}


def cast_to_bf16(src: torch.Tensor) -> torch.Tensor:
    lib = _lib.load()
    if src.dtype != torch.float32 or not src.is_contiguous():
        raise RuntimeError("cast_to_bf16 needs a contiguous fp32 tensor")
    dst = torch.empty(src.shape, dtype=torch.bfloat16, device=src.device)
    with _on_device(src.device):
        _lib.check(lib.ltr_cast_f32_to_bf16(src.data_ptr(), dst.data_ptr(), src.numel(), _stream_ptr(src.device)),
                   "ltr_cast_f32_to_bf16")
    return dst


class BlockAttentionFunction(torch.autograd.Function):
    """O = attention(q ; KV chunk table) with the recompute backward.  Inputs after the
    fixed arguments are k_0..k_{n-1}, v_0..v_{n-1}."""

    @staticmethod
    def forward(ctx, q, n_chunks, k_pos0, q_pos0, q_split, causal, scale, stepwise, out_dtype, kv_grad_acc, q_rope, *kv):
        ks, vs = list(kv[:n_chunks]), list(kv[n_chunks:])
        # fused RoPE prologue: the kernel rotates q on load and hands the rotated q back for the backward
        q_rot = torch.empty(q.shape, dtype=q.dtype, device=q.device) if q_rope is not None else None
        if stepwise:
            # one launch per ring step, merged in the epilogue into an fp32 running (O, LSE); a step brings `g` chunks of the
            # table (1, or the two half-chunks of a zig-zag rank chunk: stepwise = 2)
            g = 1 if stepwise is True else int(stepwise)
            o, lse = attn_fwd(q, ks[:g], vs[:g], k_pos0[:g], q_pos0, q_split, causal, scale, out_dtype=torch.float32,
                              q_rope=q_rope, q_rot_out=q_rot)
            for i in range(g, n_chunks, g):
                attn_fwd(q, ks[i:i + g], vs[i:i + g], k_pos0[i:i + g], q_pos0, q_split, causal, scale,
                         out=o, lse=lse, merge=True, q_rope=q_rope)
            if (out_dtype or q.dtype) != torch.float32:
                o = o.to(out_dtype or q.dtype)
        else:
            o, lse = attn_fwd(q, ks, vs, k_pos0, q_pos0, q_split, causal, scale, out_dtype=out_dtype,
                              q_rope=q_rope, q_rot_out=q_rot)
        ctx.q_rope = q_rope
        ctx.save_for_backward(q if q_rot is None else q_rot, o, lse, *kv)
        ctx.meta = (n_chunks, list(k_pos0), q_pos0, q_split, causal, scale)
        ctx.kv_grad_acc = kv_grad_acc
        ctx.mark_non_differentiable(lse)
        return o, lse

    @staticmethod
    def backward(ctx, do, _dlse):
        q, o, lse, *kv = ctx.saved_tensors
        n_chunks, k_pos0, q_pos0, q_split, causal, scale = ctx.meta
        ks, vs = kv[:n_chunks], kv[n_chunks:]
        if q.dtype not in (torch.bfloat16, torch.float32):
            raise RuntimeError("the HIP backward is implemented for bf16 and fp32 inputs")
        f32 = q.dtype == torch.float32
        if do.stride(3) != 1:
            do = do.contiguous()
        do = do.to(q.dtype)
        fuse = o.dtype == torch.bfloat16 and not f32   # DELTA computed by the dQ kernel from o
        delta = (torch.empty(lse.shape, dtype=torch.float32, device=q.device) if fuse else attn_delta(o, do))
        # one launch sees every chunk: dQ is written as bf16 by the kernel; otherwise it accumulates in fp32
        direct = n_chunks <= _lib.LTR_MAX_CHUNKS and not f32
        dq_acc = (torch.empty(q.shape, dtype=torch.bfloat16, device=q.device) if direct
                  else torch.zeros(q.shape, dtype=torch.float32, device=q.device))
        # one buffer per gradient, sliced along the sequence: every chunk's slice has the same strides.  This node's
        # q holds every query that sees these keys inside this node (autograd sums over nodes by itself), so for bf16
        # the kernels write dK / dV directly: no fp32 accumulators, no zero-fill, no cast.
        if ctx.kv_grad_acc is not None:
            # dK / dV of these chunks are summed over several nodes (the ranks of a ring) in caller-owned fp32
            # accumulators and cast once at the end, instead of one bf16 rounding per node: nothing flows to k, v here
            dk_accs, dv_accs = ctx.kv_grad_acc
            attn_bwd_accumulate(q, do, lse, delta, ks, vs, k_pos0, dq_acc, dk_accs, dv_accs, q_pos0, q_split, causal,
                                scale, o=o if fuse else None, dq_rope=ctx.q_rope)
            dq = dq_acc if (direct or f32) else cast_to_bf16(dq_acc)
            return (dq, None, None, None, None, None, None, None, None, None, None) + (None,) * (2 * n_chunks)
        lens = [k.shape[1] for k in ks]
        shape = (ks[0].shape[0], sum(lens), ks[0].shape[2], ks[0].shape[3])
        if f32:
            dk_buf = torch.zeros(shape, dtype=torch.float32, device=q.device)
            dv_buf = torch.zeros(shape, dtype=torch.float32, device=q.device)
        else:
            dk_buf = torch.empty(shape, dtype=torch.bfloat16, device=q.device)
            dv_buf = torch.empty(shape, dtype=torch.bfloat16, device=q.device)
        offs = [sum(lens[:i]) for i in range(len(lens))]
        dk_accs = [dk_buf[:, o_:o_ + n_] for o_, n_ in zip(offs, lens)]
        dv_accs = [dv_buf[:, o_:o_ + n_] for o_, n_ in zip(offs, lens)]
        attn_bwd_accumulate(q, do, lse, delta, ks, vs, k_pos0, dq_acc, dk_accs, dv_accs, q_pos0, q_split, causal, scale,
                            o=o if fuse else None, dq_rope=ctx.q_rope)
        dq = dq_acc if (direct or f32) else cast_to_bf16(dq_acc)
        dk16, dv16 = dk_buf, dv_buf
        dks = [dk16[:, o_:o_ + n_] for o_, n_ in zip(offs, lens)]
        dvs = [dv16[:, o_:o_ + n_] for o_, n_ in zip(offs, lens)]
        return (dq, None, None, None, None, None, None, None, None, None, None, *dks, *dvs)


class _PreparedCalls(threading.local):
    """Per-thread cache of filled-in argument blocks, keyed by everything but the pointers: a training loop calls with
    the same shapes, strides and positions every step, and then only the pointers are rewritten (autograd runs the
    backward on another thread than the forward, and two threads must not share one block)."""

    def __init__(self):
        self.fwd, self.bwd = {}, {}


_prepared = _PreparedCalls()
_PREPARED_MAX = 256


def _single_key(q, k, v, extra):
    return (q.shape, q.stride(), k.shape, k.stride(), v.shape, v.stride(), k.dtype, v.dtype, q.device, k.device, v.device, extra)


class SingleChunkAttentionFunction(torch.autograd.Function):
    """block_attention for its most frequent shape - ONE KV chunk, bf16, one launch (the SDPA call sites of the reference,
    model/model.py:193-198 and parallel/parallel_cp.py:224-229) - with the host work cut to what such a call needs:
    the checks are made when a geometry is first seen and the argument block is kept; later calls write five pointers
    into it.  Same kernels, same results as BlockAttentionFunction."""

    @staticmethod
    def forward(ctx, q, k, v, meta):
        k_pos0, q_pos0, q_split, causal, scale, q_rope = meta
        lib = _lib.load()
        B, Sq, Hq, D = q.shape
        dev = q.device
        o = torch.empty((B, Sq, Hq, D), dtype=torch.bfloat16, device=dev)
        lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=dev)
        q_rot = None
        key = _single_key(q, k, v, (k_pos0, q_pos0, q_split, causal, scale, None if q_rope is None else q_rope.shape[0]))
        prep = _prepared.fwd.get(key)
        if prep is None:
            for t, name in ((q, "q"), (k, "k"), (v, "v")):
                _req(t, name)
            if (k.dtype != q.dtype or v.dtype != q.dtype or k.shape != v.shape or k.shape[0] != B or k.shape[3] != D
                    or k.device != dev or v.device != dev):
                raise RuntimeError("k/v chunk shape, dtype or device mismatch")
            a = _lib.FwdArgs()
            a.B, a.Hq, a.Hkv, a.D, a.Sq = B, Hq, k.shape[2], D, Sq
            a.q_stride, a.o_stride, a.k_stride, a.v_stride = _s3(q), _s3(o), _s3(k), _s3(v)
            a.q_pos0, a.q_split = _qpos(q_pos0, Sq, q_split)
            a.scale = float(scale if scale is not None else 1.0 / math.sqrt(D))
            a.io_dtype = a.o_dtype = _lib.LTR_BF16
            a.n_chunks = 1
            a.flags = (_lib.LTR_CAUSAL if causal else 0) | (_lib.LTR_ROPE_Q if q_rope is not None else 0)
            ch = a.chunk[0]
            ch.sk, ch.pos0 = k.shape[1], int(k_pos0)
            if q_rope is not None:
                a.rope_pos0, a.rope_len = 0, q_rope.shape[0]
                a.q_rot_stride = _s3(o)          # q_rot is allocated like o: contiguous [B, Sq, Hq, D]
            if len(_prepared.fwd) >= _PREPARED_MAX:
                _prepared.fwd.clear()
            prep = _prepared.fwd[key] = (a, ch, ctypes.byref(a))
        a, ch, ref = prep
        a.q, a.o, a.lse = q.data_ptr(), o.data_ptr(), lse.data_ptr()
        ch.k, ch.v = k.data_ptr(), v.data_ptr()
        if q_rope is not None:
            _rope_table_check(q_rope, D, dev)    # the table is a per-call pointer: checked on every call
            q_rot = torch.empty((B, Sq, Hq, D), dtype=torch.bfloat16, device=dev)
            a.rope_freqs, a.q_rot = q_rope.data_ptr(), q_rot.data_ptr()
        if Sq:
            with _on_device(dev):
                rc = lib.ltr_attn_fwd(ref, _stream_ptr(dev))
            if rc:
                _lib.check(rc, "ltr_attn_fwd")
        ctx.save_for_backward(q if q_rot is None else q_rot, k, v, o, lse)
        ctx.meta = meta
        ctx.mark_non_differentiable(lse)
        return o, lse

    @staticmethod
    def backward(ctx, do, _dlse):
        q, k, v, o, lse = ctx.saved_tensors
        k_pos0, q_pos0, q_split, causal, scale, q_rope = ctx.meta
        lib = _lib.load()
        B, Sq, Hq, D = q.shape
        dev = q.device
        if do.dtype != torch.bfloat16:
            do = do.to(torch.bfloat16)
        if do.stride(3) != 1:
            do = do.contiguous()
        dq = torch.empty((B, Sq, Hq, D), dtype=torch.bfloat16, device=dev)
        dk = torch.empty(k.shape, dtype=torch.bfloat16, device=dev)
        dv = torch.empty(k.shape, dtype=torch.bfloat16, device=dev)
        if Sq == 0:
            return dq, dk.zero_(), dv.zero_(), None
        delta = torch.empty((B, Hq, Sq), dtype=torch.float32, device=dev)   # workspace: filled by the dQ kernel from o
        key = _single_key(q, k, v, (do.stride(), k_pos0, q_pos0, q_split, causal, scale, None if q_rope is None else q_rope.shape[0]))
        prep = _prepared.bwd.get(key)
        if prep is None:
            _req(do, "dO")
            a = _lib.BwdArgs()
            a.B, a.Hq, a.Hkv, a.D, a.Sq = B, Hq, k.shape[2], D, Sq
            a.q_stride, a.do_stride, a.dq_stride, a.o_stride = _s3(q), _s3(do), _s3(dq), _s3(o)
            a.k_stride, a.v_stride, a.dk_stride, a.dv_stride = _s3(k), _s3(v), _s3(dk), _s3(dv)
            a.q_pos0, a.q_split = _qpos(q_pos0, Sq, q_split)
            a.scale = float(scale if scale is not None else 1.0 / math.sqrt(D))
            a.io_dtype = _lib.LTR_BF16
            a.n_chunks = 1
            # one call holds every key these rows see and every row that sees these keys: the kernels write bf16 results
            a.flags = ((_lib.LTR_CAUSAL if causal else 0) | _lib.LTR_DQ_BF16 | _lib.LTR_DKDV_BF16 | _lib.LTR_DELTA_FROM_O
                       | (_lib.LTR_ROPE_DQ if q_rope is not None else 0))
            ch = a.chunk[0]
            ch.sk, ch.pos0 = k.shape[1], int(k_pos0)
            if q_rope is not None:
                a.rope_pos0, a.rope_len = 0, q_rope.shape[0]
            if len(_prepared.bwd) >= _PREPARED_MAX:
                _prepared.bwd.clear()
            prep = _prepared.bwd[key] = (a, ch, ctypes.byref(a))
        a, ch, ref = prep
        a.q, a.d_o, a.lse, a.delta, a.dq, a.o = q.data_ptr(), do.data_ptr(), lse.data_ptr(), delta.data_ptr(), dq.data_ptr(), o.data_ptr()
        ch.k, ch.v, ch.dk, ch.dv = k.data_ptr(), v.data_ptr(), dk.data_ptr(), dv.data_ptr()
        if q_rope is not None:
            a.rope_freqs = q_rope.data_ptr()
        with _on_device(dev):
            rc = lib.ltr_attn_bwd(ref, _stream_ptr(dev))
        if rc:
            _lib.check(rc, "ltr_attn_bwd")
        return dq, dk, dv, None


# The single-chunk bf16 call has two host sides over the same two C-ABI calls: a C++ autograd node (_ltr_node.so, built by
# lightron_amd.build: the backward then runs on the autograd thread without the interpreter) and SingleChunkAttentionFunction
# (Python).  The C++ node is used when it has been built for this ABI version and the library is the in-tree one.
USE_CPP_NODE = True
_node = None


def _cpp_node():
    global _node
    if _node is None:
        _node = False
        if not os.environ.get("LTR_ATTN_LIB"):        # the node is linked against the in-tree library
            try:
                from . import _ltr_node
                if _ltr_node.abi_version() == _lib.LTR_ABI_VERSION:
                    _node = _ltr_node
            except (ImportError, OSError):       # not built, or built against another torch: the Python node serves
                pass
    return _node


_warned_pad = False


def _padded_head_dim(q, ks, vs, k_pos0, q_pos0, q_split, causal, scale, stepwise, out_dtype, kv_grad_acc, q_rope):
    """Head dims the kernels are not instantiated for (anything but 64 and 128; the reference hands any dim // n_heads to
    SDPA, model/model.py:135, 193): a SLOW PATH that zero-pads q, k and v to the next instantiated head dim (one copy of
    each tensor per call, the gradients sliced back by autograd), keeps the scale of the TRUE head dim, and slices the
    result.  Zero columns change neither the scores nor the real columns of O.  Multiples of 8 up to 128."""
    D = q.shape[-1]
    if D > 128 or D % 8 or D <= 0:
        raise RuntimeError("head dim %d: the HIP kernels exist for 64 and 128; other head dims are zero-padded up to the "
                           "next of the two, which needs a multiple of 8 that is at most 128" % D)
    if kv_grad_acc is not None:
        raise RuntimeError("kv_grad_acc accumulators are shaped like the un-padded chunks: not available with a padded head dim")
    global _warned_pad
    if not _warned_pad:
        _warned_pad = True
        import warnings
        warnings.warn("lightron_amd: head dim %d is zero-padded to %d on every call (a copy of q, k and v)"
                      % (D, 64 if D < 64 else 128), stacklevel=3)
    Dp = 64 if D < 64 else 128
    pad = (0, Dp - D)
    lens = [k.shape[1] for k in ks]
    kbuf = torch.nn.functional.pad(ks[0] if len(ks) == 1 else torch.cat(list(ks), 1), pad)
    vbuf = torch.nn.functional.pad(vs[0] if len(vs) == 1 else torch.cat(list(vs), 1), pad)
    offs = [sum(lens[:i]) for i in range(len(lens))]
    ksp = [kbuf[:, o_:o_ + n_] for o_, n_ in zip(offs, lens)]
    vsp = [vbuf[:, o_:o_ + n_] for o_, n_ in zip(offs, lens)]
    if q_rope is not None:
        # the padded pairs are rotated by the identity (cos, sin) = (1, 0)
        ident = torch.zeros((q_rope.shape[0], (Dp - D) // 2, 2), dtype=q_rope.dtype, device=q_rope.device)
        ident[..., 0] = 1.0
        q_rope = torch.cat([q_rope, ident], 1).contiguous()
    o, lse = block_attention(torch.nn.functional.pad(q, pad), ksp, vsp, k_pos0, q_pos0, q_split, causal,
                             scale if scale is not None else 1.0 / math.sqrt(D), stepwise, out_dtype, None, q_rope)
    return o[..., :D], lse


def block_attention(q, ks, vs, k_pos0, q_pos0=0, q_split=None, causal=False, scale=None, stepwise=False,
                    out_dtype=None, kv_grad_acc=None, q_rope=None):
    """Differentiable entry: returns (O, LSE).  stepwise: False = one launch over the whole chunk table; True or an int g = one
    launch per g chunks, the partial (O, LSE) merged in the kernel's epilogue (the call pattern of a ring).  q_rope: fp32 [n_pos, D/2, 2] (cos, sin) table indexed by global
    position (layers.rope_table of precompute_freqs_cis): q is un-rotated, the forward kernel's prologue applies RoPE
    to it and the dQ kernel's epilogue the conjugate rotation, so no separate pass touches q or dQ (bf16 only).  ks are
    taken as given: rotate K once beforehand (apply_rotary_emb), it is read by every q block.  kv_grad_acc = (dk_accs, dv_accs), fp32 tensors shaped like ks / vs:
    the backward then ADDS dK / dV into them (no gradient flows to ks / vs through autograd); the owner of the
    accumulators makes the one final cast.  That is how a ring sums dK / dV over its ranks without a bf16 rounding
    per rank."""
    n = len(ks)
    if q.shape[-1] not in (64, 128):
        return _padded_head_dim(q, ks, vs, k_pos0, q_pos0, q_split, causal, scale, stepwise, out_dtype, kv_grad_acc, q_rope)
    if (n == 1 and kv_grad_acc is None and not stepwise and q.dtype == torch.bfloat16 and out_dtype in (None, torch.bfloat16)
            and q.is_cuda and ks[0].is_cuda and vs[0].is_cuda):
        if isinstance(q_pos0, (tuple, list)):
            q_pos0 = (int(q_pos0[0]), int(q_pos0[1]))
        node = _cpp_node() if USE_CPP_NODE else None
        if node:
            qa, qb = q_pos0 if isinstance(q_pos0, tuple) else (q_pos0, q_pos0)
            o, lse = node.single_chunk(q, ks[0], vs[0], int(k_pos0[0]), qa, qb, q.shape[1] if q_split is None else q_split, bool(causal),
                                       scale if scale is not None else 1.0 / math.sqrt(q.shape[3]), _stream_ptr(q.device), q_rope)
            return o, lse
        return SingleChunkAttentionFunction.apply(q, ks[0], vs[0], (int(k_pos0[0]), q_pos0, q_split, bool(causal), scale, q_rope))
    if kv_grad_acc is not None:
        dk_accs, dv_accs = kv_grad_acc
        if len(dk_accs) != n or len(dv_accs) != n:
            raise RuntimeError("kv_grad_acc needs one dK and one dV accumulator per KV chunk")
        for a, k in zip(list(dk_accs) + list(dv_accs), list(ks) + list(vs)):
            if a.dtype != torch.float32 or a.shape != k.shape:
                raise RuntimeError("kv_grad_acc entries must be fp32 tensors shaped like their chunks")
    if q_rope is not None and q.dtype != torch.bfloat16:
        raise RuntimeError("the fused RoPE prologue is implemented for bf16 q")
    return BlockAttentionFunction.apply(q, n, list(k_pos0), q_pos0, q_split, causal, scale, stepwise, out_dtype,
                                        kv_grad_acc, q_rope, *ks, *vs)
