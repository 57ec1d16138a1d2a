"""Pins the CPU oracle against things that are not retypings of its own formulas:
torch SDPA (library routine) in fp64, pure-Python brute force on tiny inputs, closed
forms and invariants.  Mirrors the reference's only acceptance test for this path
(tests/test_ring_attention.py:110-119: ring vs SDPA, max-abs < 1e-4 in fp32)."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import ring_attention_oracle as orc


def _rand(shape, seed, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * scale).to(dtype)


def _ring_all_ranks(q, k, v, W, causal, dtype=torch.float32, order=None):
    """Run the recurrence for every rank of a contiguous-sharded ring and reassemble."""
    S = q.shape[1]
    sl = S // W
    outs, lses = [], []
    for r in range(W):
        visit = orc.ring_order(r, W) if order is None else order(r)
        chunks = [(k[:, j * sl:(j + 1) * sl], v[:, j * sl:(j + 1) * sl]) for j in visit]
        kpos = [orc.contiguous_positions(j, sl) for j in visit]
        o, lse = orc.ring_attention_recurrence(q[:, r * sl:(r + 1) * sl], chunks,
                                               orc.contiguous_positions(r, sl), kpos, causal, dtype)
        outs.append(o)
        lses.append(lse)
    return torch.cat(outs, 1), torch.cat(lses, 2)


def test_reference_acceptance_noncausal_vs_sdpa():
    # the reference's own test shape: B=2, S=32, H=8, D=64, cp=4, fp32, non-causal
    q, k, v = (_rand((2, 32, 8, 64), s) for s in (1, 2, 3))
    o, _ = _ring_all_ranks(q, k, v, 4, causal=False)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)).transpose(1, 2)
    assert (o - ref).abs().max() < 1e-4


def test_config1_causal_vs_sdpa_fp64():
    # benchmark config 1: B=2 H=8 S=1024 (4x256) D=64 fp32 causal, seed 0
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn((2, 1024, 8, 64), generator=g) for _ in range(3))
    o, lse = _ring_all_ranks(q, k, v, 4, causal=True)
    qd, kd, vd = (x.double().transpose(1, 2) for x in (q, k, v))
    ref = F.scaled_dot_product_attention(qd, kd, vd, is_causal=True).transpose(1, 2)
    assert (o.double() - ref).abs().max() < 1e-4
    s = torch.einsum("bhqd,bhkd->bhqk", qd, kd) / 8.0
    s = s.masked_fill(~torch.ones(1024, 1024, dtype=torch.bool).tril(), float("-inf"))
    assert (lse.double() - torch.logsumexp(s, -1)).abs().max() < 1e-4


def test_brute_force_tiny():
    # pure-Python loops, B=1,H=1,S=6,D=2, causal, 3 chunks of 2
    q, k, v = (_rand((1, 6, 1, 2), s, torch.float64) for s in (4, 5, 6))
    o, lse = _ring_all_ranks(q, k, v, 3, causal=True, dtype=torch.float64)
    for i in range(6):
        sc = [sum(q[0, i, 0, d].item() * k[0, j, 0, d].item() for d in range(2)) / math.sqrt(2) for j in range(i + 1)]
        mx = max(sc)
        den = sum(math.exp(x - mx) for x in sc)
        assert abs(lse[0, 0, i].item() - (mx + math.log(den))) < 1e-12
        for d in range(2):
            num = sum(math.exp(sc[j] - mx) * v[0, j, 0, d].item() for j in range(i + 1))
            assert abs(o[0, i, 0, d].item() - num / den) < 1e-12


def test_closed_forms():
    # q = 0 -> uniform softmax: LSE = log(#visible keys), O = mean of visible V rows
    S, W = 16, 4
    q = torch.zeros(1, S, 2, 4, dtype=torch.float64)
    k, v = _rand((1, S, 2, 4), 7, torch.float64), _rand((1, S, 2, 4), 8, torch.float64)
    o, lse = _ring_all_ranks(q, k, v, W, causal=True, dtype=torch.float64)
    for i in range(S):
        assert abs(lse[0, 0, i].item() - math.log(i + 1)) < 1e-12
        assert (o[0, i] - v[0, :i + 1].mean(0)).abs().max() < 1e-12
    # rows are convex combinations of V rows
    q = _rand((1, S, 2, 4), 9, torch.float64)
    o, _ = _ring_all_ranks(q, k, v, W, causal=False, dtype=torch.float64)
    assert (o.amax(1) <= v.amax(1) + 1e-12).all() and (o.amin(1) >= v.amin(1) - 1e-12).all()


def test_chunking_and_order_invariance():
    q, k, v = (_rand((2, 64, 4, 16), s, torch.float64) for s in (10, 11, 12))
    base, base_lse = _ring_all_ranks(q, k, v, 1, True, torch.float64)
    for W in (2, 4, 8):
        o, lse = _ring_all_ranks(q, k, v, W, True, torch.float64)
        assert (o - base).abs().max() < 1e-12 and (lse - base_lse).abs().max() < 1e-12
        o2, _ = _ring_all_ranks(q, k, v, W, True, torch.float64, order=lambda r: list(range(W)))
        assert (o2 - base).abs().max() < 1e-12


def test_dense_matches_sdpa_and_gqa_repeat():
    q = _rand((2, 24, 8, 16), 13, torch.float64)
    k, v = _rand((2, 24, 2, 16), 14, torch.float64), _rand((2, 24, 2, 16), 15, torch.float64)
    pos = torch.arange(24)
    o, lse = orc.dense_attention(q, k, v, pos, pos, True)
    # repeat_kv semantics: each kv head repeated consecutively (model/model.py:29-33)
    kr = k[:, :, :, None, :].expand(2, 24, 2, 4, 16).reshape(2, 24, 8, 16)
    vr = v[:, :, :, None, :].expand(2, 24, 2, 4, 16).reshape(2, 24, 8, 16)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), kr.transpose(1, 2), vr.transpose(1, 2), is_causal=True)
    assert (o - ref.transpose(1, 2)).abs().max() < 1e-12
    o2, lse2 = orc.ring_attention_recurrence(q, [(k[:, :12], v[:, :12]), (k[:, 12:], v[:, 12:])], pos,
                                             [pos[:12], pos[12:]], True, torch.float64)
    assert (o2 - o).abs().max() < 1e-12 and (lse2 - lse).abs().max() < 1e-12
    assert [orc.kv_head_of(h, 4) for h in range(8)] == [0, 0, 0, 0, 1, 1, 1, 1]


def test_merge_pair_form():
    q, k, v = (_rand((1, 8, 2, 8), s, torch.float64) for s in (16, 17, 18))
    pos = torch.arange(8)
    o, lse = orc.dense_attention(q, k, v)
    o1, l1 = orc.dense_attention(q, k[:, :3], v[:, :3])
    o2, l2 = orc.dense_attention(q, k[:, 3:], v[:, 3:])
    om, lm = orc.merge_o_lse(o1, l1, o2, l2)
    assert (om - o).abs().max() < 1e-12 and (lm - lse).abs().max() < 1e-12
    # merging with an empty partial (lse = -inf, o = 0) is the identity
    om, lm = orc.merge_o_lse(o, lse, torch.zeros_like(o), torch.full_like(lse, float("-inf")))
    assert (om - o).abs().max() == 0 and (lm - lse).abs().max() == 0


def test_backward_formula_vs_autograd_sdpa():
    q = _rand((1, 20, 4, 8), 19, torch.float64)
    k, v = _rand((1, 20, 2, 8), 20, torch.float64), _rand((1, 20, 2, 8), 21, torch.float64)
    do = _rand((1, 20, 4, 8), 22, torch.float64)
    pos = torch.arange(20)
    o, lse, dq, dk, dv = orc.dense_attention_grads(q, k, v, do, pos, pos, True)
    # library routine: autograd through SDPA with materialised repeat
    qa, ka, va = (x.clone().requires_grad_(True) for x in (q, k, v))
    ref = F.scaled_dot_product_attention(qa.transpose(1, 2), ka.repeat_interleave(2, 2).transpose(1, 2),
                                         va.repeat_interleave(2, 2).transpose(1, 2), is_causal=True)
    ref.transpose(1, 2).backward(do)
    for a, b in ((dq, qa.grad), (dk, ka.grad), (dv, va.grad)):
        assert (a - b).abs().max() < 1e-10
    fq, fk, fv = orc.attention_backward_formula(q, k, v, o, lse, do, pos, pos, True, torch.float64)
    for a, b in ((fq, dq), (fk, dk), (fv, dv)):
        assert (a - b).abs().max() < 1e-10


def test_zigzag_is_a_permutation_and_balanced():
    W, S = 8, 64
    allpos = torch.cat([orc.zigzag_positions(r, W, S) for r in range(W)])
    assert sorted(allpos.tolist()) == list(range(S))
    kpos = torch.arange(S)
    counts = [orc.n_pairs_causal(orc.zigzag_positions(r, W, S), kpos) for r in range(W)]
    assert len(set(counts)) == 1 and sum(counts) == S * (S + 1) // 2
    # zig-zag ring == dense causal after un-permuting
    q, k, v = (_rand((1, S, 2, 8), s, torch.float64) for s in (23, 24, 25))
    dense, dlse = orc.dense_attention(q, k, v, kpos, kpos, True)
    for r in range(W):
        qp = orc.zigzag_positions(r, W, S)
        chunks, kp = [], []
        for j in orc.ring_order(r, W):
            p = orc.zigzag_positions(j, W, S)
            chunks.append((k[:, p], v[:, p]))
            kp.append(p)
        o, lse = orc.ring_attention_recurrence(q[:, qp], chunks, qp, kp, True, torch.float64)
        assert (o - dense[:, qp]).abs().max() < 1e-12 and (lse - dlse[:, :, qp]).abs().max() < 1e-12


def test_seq_all_to_all_bruteforce_and_roundtrip():
    W, B, Sl, H, D = 4, 2, 3, 8, 2
    full = torch.arange(B * Sl * W * H * D, dtype=torch.float32).reshape(B, Sl * W, H, D)
    shards = [full[:, r * Sl:(r + 1) * Sl] for r in range(W)]
    outs = orc.seq_all_to_all(shards, 2, 1)
    for i in range(W):  # rank i ends with the full sequence of head group i
        assert torch.equal(outs[i], full[:, :, i * (H // W):(i + 1) * (H // W)])
    back = orc.seq_all_to_all(outs, 1, 2)
    for r in range(W):
        assert torch.equal(back[r], shards[r])
    assert orc.seq_all_to_all([full], 2, 1)[0] is full


def test_rope_properties():
    D, S = 8, 40
    fc = orc.precompute_freqs_cis(D, S)
    i = torch.arange(0, D, 2).float()
    ref = torch.polar(torch.ones(S, D // 2), torch.outer(torch.arange(S), 1.0 / (10000.0 ** (i / D))).float())
    assert torch.equal(fc, ref) or (fc - ref).abs().max() < 1e-6
    x, y = _rand((1, S, 2, D), 26), _rand((1, S, 2, D), 27)
    xr, yr = orc.apply_rotary_emb(x, y, fc)
    assert torch.equal(xr[:, 0], x[:, 0])                                  # t = 0 is the identity
    pn = lambda z: z.reshape(1, S, 2, D // 2, 2).pow(2).sum(-1)
    assert (pn(xr) - pn(x)).abs().max() < 1e-5                             # pairwise norm kept
    # library routine: complex multiply on adjacent pairs
    xc = torch.view_as_complex(x.reshape(1, S, 2, D // 2, 2)) * fc[None, :, None, :]
    assert (torch.view_as_real(xc).flatten(3) - xr).abs().max() < 1e-6
    # relative-position property: <R_t q, R_s k> depends only on t - s
    qv, kv = _rand((1, 1, 1, D), 28), _rand((1, 1, 1, D), 29)
    qs, ks = orc.apply_rotary_emb(qv.expand(1, S, 1, D), kv.expand(1, S, 1, D), fc)
    d1 = (qs[0, 5, 0] * ks[0, 2, 0]).sum()
    d2 = (qs[0, 25, 0] * ks[0, 22, 0]).sum()
    assert abs(d1 - d2) < 1e-4
    # tiny hand case: D=2, t=1 -> rotation by 1 rad
    f2 = orc.precompute_freqs_cis(2, 2)
    r, _ = orc.apply_rotary_emb(torch.tensor([[[[1.0, 0.0]]], [[[1.0, 0.0]]]]).reshape(1, 2, 1, 2),
                                torch.zeros(1, 2, 1, 2), f2)
    assert abs(r[0, 1, 0, 0] - math.cos(1.0)) < 1e-6 and abs(r[0, 1, 0, 1] - math.sin(1.0)) < 1e-6


def test_fully_masked_rows_are_zero_and_minus_inf():
    q, k, v = (_rand((1, 4, 1, 4), s, torch.float64) for s in (30, 31, 32))
    o, lse = orc.ring_attention_recurrence(q, [(k, v)], torch.tensor([0, 1, 10, 11]), [torch.tensor([5, 6, 7, 8])],
                                           True, torch.float64)
    assert torch.isinf(lse[0, 0, :2]).all() and (o[0, :2] == 0).all()
    d, dl = orc.dense_attention(q, k, v, torch.tensor([0, 1, 10, 11]), torch.tensor([5, 6, 7, 8]), True)
    assert (o[0, 2:] - d[0, 2:]).abs().max() < 1e-12


def test_sampled_checks_match_dense():
    q = _rand((2, 24, 4, 8), 40, torch.float64)
    k, v = _rand((2, 24, 2, 8), 41, torch.float64), _rand((2, 24, 2, 8), 42, torch.float64)
    do = _rand((2, 24, 4, 8), 43, torch.float64)
    perm = torch.randperm(24, generator=torch.Generator().manual_seed(1))
    qpos, kpos = torch.arange(24)[perm], torch.arange(24)
    o, lse, dq, dk, dv = orc.dense_attention_grads(q[:, perm], k, v, do[:, perm], qpos, kpos, True)
    rows = [(0, 0, 3), (1, 3, 23), (0, 2, 11)]
    for (b, h, i), (ro, rl, rdq) in zip(rows, orc.sampled_rows(q[:, perm], k, v, qpos, kpos, True, rows, do[:, perm])):
        assert (ro - o[b, i, h]).abs().max() < 1e-12 and abs(rl - lse[b, h, i]) < 1e-12
        assert (rdq - dq[b, i, h]).abs().max() < 1e-12
    keys = [(0, 0, 0), (1, 1, 17), (0, 1, 23)]
    for (b, g, j), (rk, rv) in zip(keys, orc.sampled_keys(q[:, perm], k, v, o, lse, do[:, perm], qpos, kpos, True, keys)):
        assert (rk - dk[b, j, g]).abs().max() < 1e-12 and (rv - dv[b, j, g]).abs().max() < 1e-12
