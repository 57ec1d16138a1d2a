"""ltr_attn_bwd_noalloc (DELTA in the library's fixed scratch array, no allocation inside the call) against ltr_attn_bwd
with a caller-owned DELTA workspace, through the C ABI: same kernels, so the results must be bit-identical.  Two calls in
a row share the scratch array; the second is smaller, so stale rows of the first stay behind it in the array."""
import ctypes

import pytest
import torch

from oracle import ring_attention_oracle as orc

pytestmark = pytest.mark.gpu


def _case(ltr, seed, B, Hq, Hkv, D, Sq, chunk_lens, causal):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *shape: torch.randn(shape, generator=g).to(torch.bfloat16)
    Sk = sum(chunk_lens)
    q, do = mk(B, Sq, Hq, D), mk(B, Sq, Hq, D)
    k, v = mk(B, Sk, Hkv, D), mk(B, Sk, Hkv, D)
    q_pos0 = Sk - Sq
    qd, dod, kd, vd = q.cuda(), do.cuda(), k.cuda(), v.cuda()
    offs = [sum(chunk_lens[:i]) for i in range(len(chunk_lens))]
    ks = [kd[:, o:o + n] for o, n in zip(offs, chunk_lens)]
    vs = [vd[:, o:o + n] for o, n in zip(offs, chunk_lens)]
    o, lse = ltr.attn_fwd(qd, ks, vs, offs, q_pos0, None, causal)

    def run(library_scratch):
        dq = torch.empty_like(qd)
        dk = torch.zeros(B, Sk, Hkv, D, dtype=torch.float32, device="cuda")
        dv = torch.zeros_like(dk)
        dks = [dk[:, o_:o_ + n] for o_, n in zip(offs, chunk_lens)]
        dvs = [dv[:, o_:o_ + n] for o_, n in zip(offs, chunk_lens)]
        delta = None if library_scratch else torch.empty(B, Hq, Sq, dtype=torch.float32, device="cuda")
        ltr.attn_bwd_accumulate(qd, dod, lse, delta, ks, vs, offs, dq, dks, dvs, q_pos0, None, causal, o=o,
                                library_scratch=library_scratch)
        torch.cuda.synchronize()
        return dq, dk, dv

    ref = run(False)
    got = run(True)
    for a, b, name in zip(got, ref, ("dQ", "dK", "dV")):
        assert torch.equal(a, b), "%s of the no-allocation entry point differs from ltr_attn_bwd" % name
    # and both are right: the oracle, at the target's bf16 tolerance
    _, _, rdq, rdk, rdv = orc.dense_attention_grads(q, k, v, do, torch.arange(Sq) + q_pos0, torch.arange(Sk), causal)
    rel = lambda a, b: ((a.double().cpu() - b).norm() / b.norm()).item()
    assert rel(got[0], rdq) < 5e-2 and rel(got[1], rdk) < 5e-2 and rel(got[2], rdv) < 5e-2


def test_no_alloc_backward_two_calls(ltr):
    _case(ltr, 11, 2, 8, 2, 128, 640, [256, 300, 84], True)     # 10240 DELTA rows
    _case(ltr, 12, 1, 4, 4, 64, 200, [130, 70], True)           # smaller: 800 rows, stale rows behind them
    _case(ltr, 13, 1, 4, 1, 128, 96, [96], False)


def test_forward_and_no_alloc_backward_replay_in_a_hip_graph(ltr):
    """The library neither allocates nor synchronises nor records memset nodes, so one forward + backward (DELTA in the
    library's scratch array) can be captured in a HIP graph once the per-device set-up has happened in an eager call.  The
    graph is replayed on fresh inputs several times, with eager work and synchronisations between the replays, and every
    replay must give the eager call's bits."""
    B, Hq, Hkv, D, S = 2, 8, 2, 128, 384
    g = torch.Generator().manual_seed(5)
    mk = lambda h: torch.randn(B, S, h, D, generator=g).to(torch.bfloat16).cuda()
    q, k, v, do = mk(Hq), mk(Hkv), mk(Hkv), mk(Hq)
    o = torch.empty_like(q)
    lse = torch.empty(B, Hq, S, dtype=torch.float32, device="cuda")
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)      # bf16 results written by the kernels

    def step():
        ltr.attn_fwd(q, [k], [v], [0], 0, None, True, out=o, lse=lse)
        ltr.attn_bwd_accumulate(q, do, lse, None, [k], [v], [0], dq, [dk], [dv], 0, None, True, o=o, library_scratch=True)

    step()                                   # eager: per-device set-up (LDS opt-in, scratch address) happens here
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.synchronize()
    for it in range(3):
        for t in (q, k, v, do):
            t.copy_(torch.randn(t.shape, generator=g).to(torch.bfloat16))
        for t in (o, dq, dk, dv):
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (o, lse, dq, dk, dv)]
        assert all(torch.isfinite(t.float()).all() for t in got)
        step()                               # eager, same inputs
        torch.cuda.synchronize()
        for a, b, name in zip(got, (o, lse, dq, dk, dv), ("O", "LSE", "dQ", "dK", "dV")):
            assert torch.equal(a, b), "%s of replay %d differs from the eager call" % (name, it)


def test_no_alloc_rejects_what_it_cannot_hold(ltr):
    from lightron_amd import _lib as L
    lib = L.load()
    a = L.BwdArgs()
    t = torch.zeros(4096, device="cuda")
    for f in ("q", "d_o", "lse", "dq", "o"):
        setattr(a, f, t.data_ptr())
    a.B, a.Hq, a.Hkv, a.D, a.Sq, a.n_chunks = 1, 32, 8, 128, (L.LTR_NOALLOC_MAX_ROWS // 32) + 1, 1
    a.io_dtype = L.LTR_BF16
    assert lib.ltr_attn_bwd_noalloc(ctypes.byref(a), None) == -6       # LTR_ETOOBIG
    a.Sq = 64
    a.flags = L.LTR_NO_DQ
    assert lib.ltr_attn_bwd_noalloc(ctypes.byref(a), None) == -1       # the dQ kernel fills DELTA
    a.flags, a.io_dtype = 0, L.LTR_F32
    assert lib.ltr_attn_bwd_noalloc(ctypes.byref(a), None) == -2       # bf16 only
