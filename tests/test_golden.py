"""Committed golden vectors (tests/golden/vectors.npz, written by tests/golden/make_vectors.py from library SDPA in
fp64, explicit complex arithmetic and index loops - not from the oracle): the oracle is checked against them on
the CPU, the HIP path on the GPU."""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
from oracle import ring_attention_oracle as orc  # noqa: E402

G = np.load(os.path.join(ROOT, "tests", "golden", "vectors.npz"))
T = lambda name: torch.from_numpy(G[name])
BF = lambda name: torch.from_numpy(G[name]).view(torch.bfloat16)


def _ring_case_a(fwd):
    """fwd(rank, q_r, kv per rank, positions of rank) -> (o, lse) for every rank of the contiguous causal ring."""
    W = int(G["a_world"])
    q, k, v = T("a_q"), T("a_k"), T("a_v")
    Sl = q.shape[1] // W
    sl = lambda t, r: t[:, r * Sl:(r + 1) * Sl]
    for r in range(W):
        o, lse = fwd(r, W, sl(q, r), [(sl(k, j), sl(v, j)) for j in range(W)], Sl)
        assert (o.float().cpu() - sl(T("a_o"), r)).abs().max() < 1e-4
        assert (lse.float().cpu() - T("a_lse")[:, :, r * Sl:(r + 1) * Sl]).abs().max() < 1e-4


def test_oracle_recurrence_matches_golden_contiguous_ring():
    def fwd(r, W, q_r, kv, Sl):
        order = orc.ring_order(r, W)
        return orc.ring_attention_recurrence(q_r, [kv[j] for j in order], orc.contiguous_positions(r, Sl),
                                             [orc.contiguous_positions(j, Sl) for j in order], causal=True)
    _ring_case_a(fwd)


def _zigzag_shares():
    W = int(G["b_world"])
    S = G["b_q"].shape[1]
    return W, S, [orc.zigzag_positions(r, W, S) for r in range(W)]


def test_oracle_dense_and_grads_match_golden_zigzag_gqa():
    q, k, v, do = (BF(n).float() for n in ("b_q", "b_k", "b_v", "b_do"))
    W, S, shares = _zigzag_shares()
    pos = torch.arange(S)
    o, lse, dq, dk, dv = orc.dense_attention_grads(q, k, v, do, pos, pos, True)
    for got, name in ((o, "b_o"), (lse, "b_lse"), (dq, "b_dq"), (dk, "b_dk"), (dv, "b_dv")):
        assert (got.float() - T(name)).abs().max() < 1e-5, name
    # the recurrence on each zig-zag share (own half-chunks first, then the ring order) gives the same rows
    for r in range(W):
        order = orc.ring_order(r, W)
        kv = [(k[:, shares[j]], v[:, shares[j]]) for j in order]
        o_r, lse_r = orc.ring_attention_recurrence(q[:, shares[r]], kv, shares[r], [shares[j] for j in order], causal=True)
        assert (o_r - T("b_o")[:, shares[r]]).abs().max() < 1e-4
        assert (lse_r - T("b_lse")[:, :, shares[r]]).abs().max() < 1e-4


def test_oracle_rope_and_exchange_match_golden():
    x, p0 = T("c_x"), int(G["c_pos0"])
    fc = orc.precompute_freqs_cis(x.shape[-1], p0 + x.shape[1])[p0:]
    y, _ = orc.apply_rotary_emb(x, x, fc)
    assert (y - T("c_y")).abs().max() < 1e-4        # fp32 angles near 100 rad: the table itself carries ~1e-5
    shards = T("d_in")
    out = orc.seq_all_to_all([shards[r] for r in range(shards.shape[0])], 2, 1)
    assert torch.equal(torch.stack(out, 0), T("d_out"))


@pytest.mark.gpu
def test_hip_ring_matches_golden_contiguous_fp32(ltr):
    def fwd(r, W, q_r, kv, Sl):
        ring = ltr.LocalRing(r, W, kv=[(a.cuda(), b.cuda()) for a, b in kv], causal=True)
        o, lse = ltr.ring_attention_with_lse(q_r.cuda(), kv[r][0].cuda(), kv[r][1].cuda(), ring)
        return o, lse
    _ring_case_a(fwd)


@pytest.mark.gpu
def test_hip_zigzag_gqa_forward_backward_matches_golden(ltr):
    q, k, v, do = (BF(n) for n in ("b_q", "b_k", "b_v", "b_do"))
    W, S, shares = _zigzag_shares()
    hc = S // (2 * W)
    dk_acc = torch.zeros(k.shape, dtype=torch.float32, device="cuda")
    dv_acc = torch.zeros_like(dk_acc)
    kd, vd = k.cuda(), v.cuda()
    halves = [slice(i * hc, (i + 1) * hc) for i in range(2 * W)]
    ks, vs, pos0 = [kd[:, h] for h in halves], [vd[:, h] for h in halves], [i * hc for i in range(2 * W)]
    rel = lambda a, b: ((a.float().cpu() - b).norm() / b.norm()).item()
    for r in range(W):
        qr, dor = q[:, shares[r]].contiguous().cuda(), do[:, shares[r]].contiguous().cuda()
        qp = (r * hc, (2 * W - 1 - r) * hc)
        o, lse = ltr.attn_fwd(qr, ks, vs, pos0, qp, hc, True)
        assert (o.float().cpu() - T("b_o")[:, shares[r]]).abs().max() < 2e-2
        assert (lse.cpu() - T("b_lse")[:, :, shares[r]]).abs().max() < 1e-2
        delta = ltr.attn_delta(o, dor)
        dq_acc = torch.zeros(qr.shape, dtype=torch.float32, device="cuda")
        ltr.attn_bwd_accumulate(qr, dor, lse, delta, ks, vs, pos0, dq_acc, [dk_acc[:, h] for h in halves],
                                [dv_acc[:, h] for h in halves], qp, hc, True)
        assert rel(dq_acc, T("b_dq")[:, shares[r]]) < 5e-2
    assert rel(dk_acc, T("b_dk")) < 5e-2 and rel(dv_acc, T("b_dv")) < 5e-2


@pytest.mark.gpu
def test_hip_rope_and_exchange_match_golden(ltr):
    x, p0 = T("c_x"), int(G["c_pos0"])
    # head dim 16 is a multiple of 8: the kernel path; table from the product's own precompute_freqs_cis
    fc = ltr.precompute_freqs_cis(x.shape[-1], p0 + x.shape[1])[p0:]
    y, _ = ltr.apply_rotary_emb(x.cuda(), x.cuda(), fc.cuda())
    assert (y.cpu() - T("c_y")).abs().max() < 1e-4
    shards = T("d_in").cuda()
    out = ltr._all_to_all(shards, 2, 1, ltr.LocalCPGroup(shards.shape[0]))
    assert torch.equal(out.cpu(), T("d_out"))
