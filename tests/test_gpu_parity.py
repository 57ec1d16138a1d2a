"""GPU parity tests: the HIP path (through the C ABI) against the CPU oracle on the same
seeded inputs.  Tolerances are the ones the target states: fp32 max-abs <= 1e-4 on O and
LSE; bf16 <= 2e-2 max-abs on O and <= 5e-2 relative (per-tensor norm) on dQ/dK/dV."""
import math

import pytest
import torch

from oracle import ring_attention_oracle as orc

pytestmark = pytest.mark.gpu

O_TOL_BF16 = 2e-2
LSE_TOL_BF16 = 2e-2
GRAD_RTOL_BF16 = 5e-2
F32_TOL = 1e-4


def _randn(shape, gen, dtype, scale=1.0):
    return (torch.randn(shape, generator=gen, dtype=torch.float32) * scale).to(dtype)


def _rel(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-30)).item()


def _dev(*ts):
    return [t.cuda() for t in ts]


@pytest.mark.parametrize("D,Hq,Hkv,Sq,Sk,causal", [
    (128, 2, 2, 256, 256, False),
    (128, 4, 1, 128, 320, True),
    (64, 2, 2, 192, 192, True),
    (128, 2, 2, 100, 77, False),      # ragged: tails in both dimensions
    (64, 4, 2, 33, 130, True),
])
def test_fwd_single_chunk_bf16(ltr, D, Hq, Hkv, Sq, Sk, causal):
    g = torch.Generator().manual_seed(100 + Sq + Sk)
    q = _randn((2, Sq, Hq, D), g, torch.bfloat16)
    k = _randn((2, Sk, Hkv, D), g, torch.bfloat16)
    v = _randn((2, Sk, Hkv, D), g, torch.bfloat16)
    q_pos0 = Sk - Sq if causal and Sk >= Sq else 0     # bottom-right aligned when Sk > Sq
    qd, kd, vd = _dev(q, k, v)
    o, lse = ltr.attn_fwd(qd, [kd], [vd], [0], q_pos0, None, causal)
    ro, rlse = orc.dense_attention(q, k, v, torch.arange(Sq) + q_pos0, torch.arange(Sk), causal)
    fin = torch.isfinite(rlse)
    assert (o.cpu().double() - ro).abs().max() < O_TOL_BF16
    assert torch.equal(torch.isfinite(lse.cpu()), fin)
    assert (lse.cpu().double()[fin] - rlse[fin]).abs().max() < LSE_TOL_BF16


def test_config1_fp32_ring_four_ranks(ltr):
    """benchmark config 1: B=2 H=8 S=1024 as 4 x 256, D=64, fp32, causal, seed 0, forward."""
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn((2, 8, 1024, 64), generator=g) for _ in range(3))   # [B,H,S,D] as stated
    qs, ks, vs = (x.transpose(1, 2) for x in (q, k, v))                        # views [B,S,H,D]
    W, sl = 4, 256
    pos = torch.arange(1024)
    ro, rlse = orc.dense_attention(qs, ks, vs, pos, pos, True)
    kd, vd, qd = ks.cuda(), vs.cuda(), qs.cuda()
    for stepwise in (False, True):
        outs, lses = [], []
        for r in range(W):
            kv = [(kd[:, j * sl:(j + 1) * sl], vd[:, j * sl:(j + 1) * sl]) for j in range(W)]
            ring = ltr.LocalRing(r, W, kv, causal=True, stepwise=stepwise)
            o = ltr.ring_attention_kernel(qd[:, r * sl:(r + 1) * sl], kv[r][0], kv[r][1], ring, None)
            outs.append(o.cpu())
            lses.append(ring.last_lse.cpu())
            # the oracle's recurrence in the reference's visiting order, same rank
            oo, ol = orc.ring_attention_recurrence(
                qs[:, r * sl:(r + 1) * sl], [(ks[:, j * sl:(j + 1) * sl], vs[:, j * sl:(j + 1) * sl]) for j in ring.order()],
                orc.contiguous_positions(r, sl), [orc.contiguous_positions(j, sl) for j in ring.order()], True)
            assert (o.cpu() - oo).abs().max() < F32_TOL and (ring.last_lse.cpu() - ol).abs().max() < F32_TOL
        o = torch.cat(outs, 1)
        lse = torch.cat(lses, 2)
        assert o.shape == (2, 1024, 8, 64) and lse.shape == (2, 8, 1024)
        assert (o.double() - ro).abs().max() < F32_TOL
        assert (lse.double() - rlse).abs().max() < F32_TOL


def test_reference_acceptance_noncausal_fp32(ltr):
    """The reference's own test: B=2 S=32 H=8 D=64 fp32 non-causal, cp=4, vs SDPA, < 1e-4
    (tests/test_ring_attention.py:31-37, 110-119)."""
    g = torch.Generator().manual_seed(1)
    q, k, v = (torch.randn((2, 32, 8, 64), generator=g) for _ in range(3))
    ref = torch.nn.functional.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2),
                                                           v.transpose(1, 2)).transpose(1, 2)
    qd, kd, vd = _dev(q, k, v)
    outs = []
    for r in range(4):
        kv = [(kd[:, j * 8:(j + 1) * 8], vd[:, j * 8:(j + 1) * 8]) for j in range(4)]
        outs.append(ltr.ring_attention_kernel(qd[:, r * 8:(r + 1) * 8], kv[r][0], kv[r][1], ltr.LocalRing(r, 4, kv), None))
    assert (torch.cat(outs, 1).cpu() - ref).abs().max() < F32_TOL


@pytest.mark.parametrize("D,B,Hq,Hkv,Sq,q_pos,split,chunks,causal,want", [
    (64, 2, 8, 8, 256, (768, 768), None, [(768, 256), (512, 256), (256, 256), (0, 256)], True, "fwd_f32_mfma_kernel<64, 4>"),   # config 1, rank 3
    (64, 2, 8, 8, 8, (0, 0), None, [(0, 8), (24, 8), (16, 8), (8, 8)], False, "fwd_f32_mfma_kernel<64, 4>"),   # the reference's acceptance shape
    (64, 4, 16, 4, 300, (100, 900), 130, [(0, 200), (200, 333), (533, 700)], True, "fwd_f32_mfma_kernel<64, 2>"),   # ragged, GQA, two-segment rows
    (64, 2, 16, 16, 1024, (0, 0), None, [(0, 1024)], True, "fwd_f32_mfma_kernel<64, 1>"),
    (128, 1, 4, 2, 200, (56, 56), None, [(0, 100), (100, 156)], True, "fwd_f32_mfma_kernel<128, 2>"),
    (128, 4, 16, 4, 520, (0, 0), None, [(0, 260), (260, 300)], False, "fwd_f32_mfma_kernel<128, 1>"),
])
def test_fp32_forward_on_the_matrix_pipe(ltr, D, B, Hq, Hkv, Sq, q_pos, split, chunks, causal, want):
    """The fp32 forward on v_mfma_f32_32x32x2_f32 in every instantiation (1, 2 or 4 key shares per row group, chosen by
    the library from the launch's rows: the plan must name the expected kernel on a 256-CU device), against the dense
    oracle to 1e-4 on O and LSE, in one launch and step by step with the merge epilogue, and against the scalar fp32
    kernel (LTR_FWD_F32_SCALAR)."""
    plan = ltr.attn_plan(B, Hq, Hkv, D, Sq, [n for _, n in chunks], [p0 for p0, _ in chunks], q_pos, split, causal, dtype=torch.float32)
    if plan["compute_units"] == 256:
        assert plan["fwd"]["kernel"] == want
    assert plan["fwd"]["kernel"].startswith("fwd_f32_mfma_kernel")
    assert ltr.attn_plan(B, Hq, Hkv, D, Sq, [n for _, n in chunks], [p0 for p0, _ in chunks], q_pos, split, causal,
                         dtype=torch.float32, f32_scalar=True)["fwd"]["kernel"] == "fwd_f32_kernel<%d>" % D
    g = torch.Generator().manual_seed(4000 + Sq + D)
    sp = Sq if split is None else split
    qpos = torch.cat([torch.arange(sp) + q_pos[0], torch.arange(Sq - sp) + q_pos[1]])
    q = _randn((B, Sq, Hq, D), g, torch.float32)
    ks = [_randn((B, n, Hkv, D), g, torch.float32) for _, n in chunks]
    vs = [_randn((B, n, Hkv, D), g, torch.float32) for _, n in chunks]
    kpos = torch.cat([torch.arange(n) + p0 for p0, n in chunks])
    o_ref, lse_ref = orc.dense_attention(q, torch.cat(ks, 1), torch.cat(vs, 1), qpos, kpos, causal)
    qd, kd, vd = q.cuda(), [k.cuda() for k in ks], [v.cuda() for v in vs]
    pos0 = [p0 for p0, _ in chunks]
    o, lse = ltr.attn_fwd(qd, kd, vd, pos0, q_pos, split, causal)
    o_sc, lse_sc = ltr.attn_fwd(qd, kd, vd, pos0, q_pos, split, causal, f32_scalar=True)
    o_st, lse_st = ltr.attn_fwd(qd, kd[:1], vd[:1], pos0[:1], q_pos, split, causal)
    for i in range(1, len(chunks)):
        ltr.attn_fwd(qd, kd[i:i + 1], vd[i:i + 1], pos0[i:i + 1], q_pos, split, causal, out=o_st, lse=lse_st, merge=True)
    fin = torch.isfinite(lse_ref)
    for oo, ll in ((o, lse), (o_sc, lse_sc), (o_st, lse_st)):
        assert (oo.cpu().double() - o_ref).abs().max() < F32_TOL
        assert torch.equal(torch.isfinite(ll.cpu()), fin)
        assert (ll.cpu().double()[fin] - lse_ref[fin]).abs().max() < F32_TOL
    assert (o - o_sc).abs().max() < 2e-5


@pytest.mark.parametrize("with_rope", [False, True])
def test_single_chunk_host_sides_agree(ltr, with_rope):
    """The single-chunk bf16 call through the C++ autograd node (_ltr_node.so) and through the Python autograd Function:
    same two C-ABI calls, so O, LSE and all three gradients must be bit-identical; GQA, strided [B,H,S,D] views, a
    non-contiguous dO, with and without the fused RoPE prologue; and the result against the dense oracle."""
    from lightron_amd import attention as A
    assert A._cpp_node(), "the C++ autograd node has not been built (python -m lightron_amd.build)"
    g = torch.Generator().manual_seed(91)
    B, S, Hq, Hkv, D = 2, 200, 8, 2, 64
    q = _randn((B, Hq, S, D), g, torch.bfloat16).transpose(1, 2)
    k = _randn((B, Hkv, S, D), g, torch.bfloat16).transpose(1, 2)
    v = _randn((B, S, Hkv, D), g, torch.bfloat16)
    do = _randn((B, Hq, S, D), g, torch.bfloat16).transpose(1, 2)
    table = ltr.rope_table(ltr.precompute_freqs_cis(D, S, device="cuda")) if with_rope else None
    res = []
    for use_cpp in (True, False):
        A.USE_CPP_NODE = use_cpp
        try:
            qd, kd, vd = (x.cuda().requires_grad_(True) for x in (q, k, v))
            o, lse = ltr.block_attention(qd, [kd], [vd], [0], 0, None, causal=True, q_rope=table)
            assert type(o.grad_fn).__name__ == ("CppFunction" if use_cpp else "SingleChunkAttentionFunctionBackward")
            assert ("SingleChunkNode" in o.grad_fn.name()) == use_cpp
            o.backward(do.cuda())
            res.append((o.detach(), lse, qd.grad, kd.grad, vd.grad))
        finally:
            A.USE_CPP_NODE = True
    for a, b in zip(*res):
        assert torch.equal(a, b)
    if not with_rope:
        pos = torch.arange(S)
        ro, rlse, rdq, rdk, rdv = orc.dense_attention_grads(q.float(), k.float(), v.float(), do.float(), pos, pos, True, dtype=torch.float32)
        o, lse, dq, dk, dv = (x.cpu() for x in res[0])
        assert (o.float() - ro).abs().max() < O_TOL_BF16 and (lse - rlse).abs().max() < LSE_TOL_BF16
        assert _rel(dq, rdq) < GRAD_RTOL_BF16 and _rel(dk, rdk) < GRAD_RTOL_BF16 and _rel(dv, rdv) < GRAD_RTOL_BF16


def test_config2_shape_scaled_multi_chunk_bf16(ltr):
    """Config 2 at reduced B/H: last rank's Q chunk of 1024 against 8 KV chunks of 1024, bf16, causal,
    inputs N(0,1)*0.5, fused and step-wise (merge epilogue) paths."""
    g = torch.Generator().manual_seed(0)
    B, H, D, sl, W = 1, 4, 128, 1024, 8
    q = _randn((B, sl, H, D), g, torch.bfloat16, 0.5)
    ks = [_randn((B, sl, H, D), g, torch.bfloat16, 0.5) for _ in range(W)]
    vs = [_randn((B, sl, H, D), g, torch.bfloat16, 0.5) for _ in range(W)]
    kall, vall = torch.cat(ks, 1), torch.cat(vs, 1)
    ro, rlse = orc.dense_attention(q, kall, vall, torch.arange(sl) + 7 * sl, torch.arange(W * sl), True)
    kv = [(k.cuda(), v.cuda()) for k, v in zip(ks, vs)]
    for stepwise in (False, True):
        ring = ltr.LocalRing(7, W, kv, causal=True, stepwise=stepwise)
        o = ltr.ring_attention_kernel(q.cuda(), kv[7][0], kv[7][1], ring, None)
        assert o.dtype == torch.bfloat16
        assert (o.cpu().double() - ro).abs().max() < O_TOL_BF16
        assert (ring.last_lse.cpu().double() - rlse).abs().max() < LSE_TOL_BF16


def _grads_case(ltr, B, Hq, Hkv, D, S, W, layout, causal, seed, dist="normal", dtype=torch.bfloat16):
    """Every rank of a ring: forward and backward, dK/dV summed over ranks, vs dense autograd."""
    g = torch.Generator().manual_seed(seed)
    if dist == "normal":
        mk = lambda shape: _randn(shape, g, dtype)
    else:
        mk = lambda shape: (torch.rand(shape, generator=g) * 2 - 1).to(dtype)
    o_tol, lse_tol, g_tol = ((O_TOL_BF16, LSE_TOL_BF16, GRAD_RTOL_BF16) if dtype == torch.bfloat16
                             else (F32_TOL, F32_TOL, F32_TOL))
    q, k, v, do = mk((B, S, Hq, D)), mk((B, S, Hkv, D)), mk((B, S, Hkv, D)), mk((B, S, Hq, D))
    pos = torch.arange(S)
    ro, rlse, rdq, rdk, rdv = orc.dense_attention_grads(q, k, v, do, pos, pos, causal)
    if layout == "zigzag":
        rank_pos = [orc.zigzag_positions(r, W, S) for r in range(W)]
    else:
        rank_pos = [orc.contiguous_positions(r, S // W) for r in range(W)]
    qd, kd, vd, dod = _dev(q, k, v, do)
    kl = [kd[:, p.cuda()].clone().requires_grad_(True) for p in rank_pos]
    vl = [vd[:, p.cuda()].clone().requires_grad_(True) for p in rank_pos]
    o = torch.empty_like(qd)
    dq = torch.empty_like(qd)
    lse = torch.empty(B, Hq, S)
    for r in range(W):
        ql = qd[:, rank_pos[r].cuda()].clone().requires_grad_(True)
        ring = ltr.LocalRing(r, W, list(zip(kl, vl)), causal=causal, layout=layout)
        out = ltr.ring_attention_kernel(ql, kl[r], vl[r], ring, None)
        out.backward(dod[:, rank_pos[r].cuda()])
        o[:, rank_pos[r].cuda()] = out.detach()
        dq[:, rank_pos[r].cuda()] = ql.grad
        lse[:, :, rank_pos[r]] = ring.last_lse.cpu()
    dk = torch.empty_like(kd)
    dv = torch.empty_like(vd)
    for r in range(W):
        dk[:, rank_pos[r].cuda()] = kl[r].grad
        dv[:, rank_pos[r].cuda()] = vl[r].grad
    assert (o.cpu().double() - ro).abs().max() < o_tol
    assert (lse.double() - rlse).abs().max() < lse_tol
    for name, a, b in (("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
        assert a.dtype == dtype
        assert _rel(a.cpu(), b) < g_tol, (name, _rel(a.cpu(), b))
        if dtype == torch.float32:
            assert (a.cpu().double() - b).abs().max() < F32_TOL * max(1.0, b.abs().max().item()), name


def test_config3_shape_scaled_gqa_zigzag_fwd_bwd(ltr):
    """Config 3 at reduced S: GQA 8/2, D=128, zig-zag over 4 ranks, causal, N(0,1), seed 0."""
    _grads_case(ltr, 1, 8, 2, 128, 1024, 4, "zigzag", True, 0)


def test_contiguous_ring_mha_fwd_bwd(ltr):
    _grads_case(ltr, 2, 2, 2, 128, 512, 2, "contiguous", True, 3)


def test_noncausal_d64_fwd_bwd(ltr):
    """Config 5's kernel case at reduced size: non-causal, D=64, U(-1,1), seed 7."""
    _grads_case(ltr, 2, 4, 4, 64, 384, 1, "contiguous", False, 7, dist="uniform")


def test_config1_fp32_ring_fwd_bwd(ltr):
    """Config 1's shape (B=2, H=8, S=1024 as 4 ranks x 256, D=64, fp32, causal) through the fp32 backward kernels:
    O, LSE and all three gradients to 1e-4."""
    _grads_case(ltr, 2, 8, 8, 64, 1024, 4, "contiguous", True, 0, dtype=torch.float32)


@pytest.mark.parametrize("D,B,Hq,Hkv,Sq,q_pos,split,chunks,causal", [
    (64, 2, 8, 8, 256, (768, 768), None, [(768, 256), (512, 256), (256, 256), (0, 256)], True),     # config 1, rank 3: 4 key shares
    (64, 4, 16, 4, 300, (100, 900), 130, [(0, 200), (200, 333), (533, 700)], True),                 # ragged, GQA, two-segment rows
    (64, 2, 16, 16, 1024, (0, 0), None, [(0, 1024)], True),                                          # one key share
    (128, 1, 4, 2, 200, (56, 56), None, [(0, 100), (100, 156)], True),
    (128, 4, 16, 4, 520, (0, 0), None, [(0, 260), (260, 300)], False),
])
def test_fp32_backward_on_the_matrix_pipe(ltr, D, B, Hq, Hkv, Sq, q_pos, split, chunks, causal):
    """The fp32 backward on v_mfma_f32_32x32x2_f32 (bwd_dq_f32_mfma_kernel in its key-share instantiations,
    bwd_dkdv_f32_mfma_kernel) against dense fp64 autograd to 1e-4 relative per tensor, and against the scalar fp32 kernels
    (LTR_BWD_F32_SCALAR); accumulation over two calls (the accumulators are added to, not overwritten)."""
    lens, pos0 = [n for _, n in chunks], [p0 for p0, _ in chunks]
    plan = ltr.attn_plan(B, Hq, Hkv, D, Sq, lens, pos0, q_pos, split, causal, dtype=torch.float32)
    assert plan["dq"]["kernel"].startswith("bwd_dq_f32_mfma_kernel") and plan["dkdv"]["kernel"] == "bwd_dkdv_f32_mfma_kernel<%d>" % D
    g = torch.Generator().manual_seed(4100 + Sq + D)
    sp = Sq if split is None else split
    qpos = torch.cat([torch.arange(sp) + q_pos[0], torch.arange(Sq - sp) + q_pos[1]])
    q, do = _randn((B, Sq, Hq, D), g, torch.float32), _randn((B, Sq, Hq, D), g, torch.float32)
    kbuf, vbuf = _randn((B, sum(lens), Hkv, D), g, torch.float32), _randn((B, sum(lens), Hkv, D), g, torch.float32)
    kpos = torch.cat([torch.arange(n) + p0 for p0, n in chunks])
    ro, rlse, rdq, rdk, rdv = orc.dense_attention_grads(q, kbuf, vbuf, do, qpos, kpos, causal)
    qd, dod, kd, vd = q.cuda(), do.cuda(), kbuf.cuda(), vbuf.cuda()
    offs = [sum(lens[:i]) for i in range(len(lens))]
    ks = [kd[:, o_:o_ + n_] for o_, n_ in zip(offs, lens)]
    vs = [vd[:, o_:o_ + n_] for o_, n_ in zip(offs, lens)]
    o, lse = ltr.attn_fwd(qd, ks, vs, pos0, q_pos, split, causal)
    delta = ltr.attn_delta(o, dod)
    res = {}
    for scalar in (False, True):
        dq = torch.zeros_like(qd)
        dk, dv = torch.zeros_like(kd), torch.zeros_like(vd)
        dks = [dk[:, o_:o_ + n_] for o_, n_ in zip(offs, lens)]
        dvs = [dv[:, o_:o_ + n_] for o_, n_ in zip(offs, lens)]
        for _ in range(2):      # two calls: every gradient must come out doubled
            ltr.attn_bwd_accumulate(qd, dod, lse, delta, ks, vs, pos0, dq, dks, dvs, q_pos, split, causal, f32_scalar=scalar)
        res[scalar] = (dq.cpu() / 2, dk.cpu() / 2, dv.cpu() / 2)
    for got, ref in zip(res[False], (rdq, rdk, rdv)):
        assert _rel(got, ref) < 1e-4
    for a, b in zip(res[False], res[True]):
        assert _rel(a, b) < 2e-5


def test_fp32_gqa_zigzag_d128_fwd_bwd(ltr):
    _grads_case(ltr, 1, 4, 2, 128, 512, 4, "zigzag", True, 5, dtype=torch.float32)


def test_fp32_noncausal_fwd_bwd(ltr):
    _grads_case(ltr, 2, 2, 1, 64, 192, 1, "contiguous", False, 9, dist="uniform", dtype=torch.float32)


@pytest.mark.parametrize("seed", list(range(10)))
def test_fp32_backward_random_shapes(ltr, seed):
    """Ragged sizes, several KV chunks with gaps in their positions, GQA, rows that see no key: the fp32 backward against
    dense fp64 autograd, 1e-4 relative per tensor."""
    import random
    rnd = random.Random(9000 + seed)
    g = torch.Generator().manual_seed(9500 + seed)
    D = rnd.choice([64, 128])
    Hkv = rnd.choice([1, 2])
    Hq = Hkv * rnd.choice([1, 3])
    B = rnd.choice([1, 2])
    Sq = rnd.choice([1, 31, 64, 65, 100, 150])
    n_ch = rnd.randint(1, 3)
    sks = [rnd.choice([1, 17, 64, 70, 129]) for _ in range(n_ch)]
    causal = rnd.random() < 0.7
    starts, p = [], rnd.randint(0, 20)
    for sk in sks:
        starts.append(p)
        p += sk + rnd.choice([0, 0, 5])
    qp = rnd.randint(0, p)
    q_pos = torch.arange(qp, qp + Sq)
    q, do = _randn((B, Sq, Hq, D), g, torch.float32), _randn((B, Sq, Hq, D), g, torch.float32)
    kbuf, vbuf = _randn((B, sum(sks), Hkv, D), g, torch.float32), _randn((B, sum(sks), Hkv, D), g, torch.float32)
    offs = [sum(sks[:i]) for i in range(n_ch)]
    k_pos = torch.cat([torch.arange(starts[i], starts[i] + sks[i]) for i in range(n_ch)])
    ro, rlse, rdq, rdk, rdv = orc.dense_attention_grads(q, kbuf, vbuf, do, q_pos, k_pos, causal)
    qd = q.cuda().requires_grad_(True)
    kd, vd = kbuf.cuda().requires_grad_(True), vbuf.cuda().requires_grad_(True)
    ks = [kd[:, offs[i]:offs[i] + sks[i]] for i in range(n_ch)]
    vs = [vd[:, offs[i]:offs[i] + sks[i]] for i in range(n_ch)]
    o, lse = ltr.block_attention(qd, ks, vs, starts, qp, None, causal=causal)
    o.backward(do.cuda())
    assert (o.detach().cpu().double() - ro).abs().max() < F32_TOL
    for name, a, b in (("dq", qd.grad, rdq), ("dk", kd.grad, rdk), ("dv", vd.grad, rdv)):
        assert a.dtype == torch.float32
        assert torch.isfinite(a).all(), name
        # (a single visible key gives dS = P (dP - DELTA) = 0 exactly: only an absolute bound makes sense there)
        if b.abs().max() > 1e-3:
            assert _rel(a.cpu(), b) < F32_TOL, (name, _rel(a.cpu(), b))
        else:
            assert (a.cpu().double() - b).abs().max() < F32_TOL, name


def test_ragged_bwd(ltr):
    g = torch.Generator().manual_seed(11)
    B, Hq, Hkv, D, Sq, Sk = 1, 4, 2, 128, 75, 201
    q, do = _randn((B, Sq, Hq, D), g, torch.bfloat16), _randn((B, Sq, Hq, D), g, torch.bfloat16)
    k, v = _randn((B, Sk, Hkv, D), g, torch.bfloat16), _randn((B, Sk, Hkv, D), g, torch.bfloat16)
    qpos, kpos = torch.arange(Sq) + 100, torch.arange(Sk)
    ro, rlse, rdq, rdk, rdv = orc.dense_attention_grads(q, k, v, do, qpos, kpos, True)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o, lse = ltr.block_attention(qd, [kd], [vd], [0], 100, None, True)
    o.backward(do.cuda())
    assert (o.detach().cpu().double() - ro).abs().max() < O_TOL_BF16
    for a, b in ((qd.grad, rdq), (kd.grad, rdk), (vd.grad, rdv)):
        assert _rel(a.cpu(), b) < GRAD_RTOL_BF16


def test_fully_masked_rows(ltr):
    """Queries that precede every key: O = 0, LSE = -inf, and merging keeps a later partial intact."""
    g = torch.Generator().manual_seed(12)
    q, k, v = (_randn((1, 64, 2, 128), g, torch.bfloat16).cuda() for _ in range(3))
    o, lse = ltr.attn_fwd(q, [k], [v], [1000], 0, None, True)
    assert torch.isinf(lse).all() and (lse < 0).all() and (o == 0).all()
    o2, lse2 = ltr.attn_fwd(q, [k], [v], [0], 0, None, True, out_dtype=torch.float32)
    ref = o2.clone()
    ltr.attn_fwd(q, [k], [v], [1000], 0, None, True, out=o2, lse=lse2, merge=True)
    assert torch.equal(o2, ref)


def test_strided_bhsd_views(ltr):
    """[B,H,S,D] storage passed as transposed views gives the same result as [B,S,H,D] storage."""
    g = torch.Generator().manual_seed(13)
    q, k, v = (_randn((2, 128, 4, 128), g, torch.bfloat16).cuda() for _ in range(3))
    o1, l1 = ltr.attn_fwd(q, [k], [v], [0], 0, None, True)
    qt, kt, vt = (x.transpose(1, 2).contiguous().transpose(1, 2) for x in (q, k, v))
    assert qt.stride() != q.stride()
    o2, l2 = ltr.attn_fwd(qt, [kt], [vt], [0], 0, None, True)
    assert torch.equal(o1, o2) and torch.equal(l1, l2)


def test_cast_kernel(ltr):
    x = torch.randn(1000003, generator=torch.Generator().manual_seed(14)).cuda()[:1000001]
    x = x.clone()
    assert torch.equal(ltr.cast_to_bf16(x), x.to(torch.bfloat16))


@pytest.mark.parametrize("W,B,Sl,H,D,dtype", [(4, 2, 64, 8, 64, torch.bfloat16), (2, 1, 50, 2, 128, torch.bfloat16),
                                              (3, 1, 40, 6, 64, torch.bfloat16), (8, 1, 32, 8, 64, torch.bfloat16),
                                              (2, 1, 50, 2, 128, torch.float32), (4, 2, 32, 4, 64, torch.float32)])
def test_ulysses_module_matches_oracle(ltr, W, B, Sl, H, D, dtype):
    """Config 5's layout at reduced size (and other ring sizes / ragged shard lengths): W ranks, sequence shards
    [B, S/W, H, D] -> head shards, attention, and back; literal (exchange-by-exchange) and zero-copy paths vs the
    oracle."""
    import torch.nn as nn
    dim = H * D

    class Attn(nn.Module):
        def __init__(self):
            super().__init__()
            self.n_heads = H
            self.wq, self.wk, self.wv, self.wo = (nn.Linear(dim, dim, bias=False) for _ in range(4))

    class Args:
        n_heads, tp_size = H, 1
    Args.dim = dim
    torch.manual_seed(7)
    attn = Attn().to(dtype)
    x = ((torch.rand(W, B, Sl, dim) * 2 - 1) * 0.5).to(dtype)
    y_tol, g_tol = (3e-2, 5e-2) if dtype == torch.bfloat16 else (2e-4, 2e-4)
    fc = orc.precompute_freqs_cis(D, W * Sl)
    # oracle: projections in fp32 torch on the CPU, exchange, RoPE, dense causal attention, exchange back; with
    # autograd, so that the gradients of the input and of the four weights are checked as well
    dy = ((torch.rand(W, B, Sl, dim) * 2 - 1) * 0.1).to(dtype)
    ws = {n: p_.detach().float().clone().requires_grad_(True) for n, p_ in attn.named_parameters()}
    xr = x.float().clone().requires_grad_(True)
    xq, xk, xv = ((xr @ ws[n].T).view(W, B, Sl, H, D) for n in ("wq.weight", "wk.weight", "wv.weight"))
    sq, sk, sv = (orc.seq_all_to_all([t[r] for r in range(W)], 2, 1) for t in (xq, xk, xv))
    outs = []
    pos = torch.arange(W * Sl)
    for r in range(W):
        rq, rk = orc.apply_rotary_emb(sq[r], sk[r], fc)
        o, _ = orc.dense_attention(rq, rk, sv[r], pos, pos, True)
        outs.append(o.float())
    back = orc.seq_all_to_all(outs, 1, 2)
    ref = torch.stack([b_.flatten(2) @ ws["wo.weight"].T for b_ in back], 0)
    ref.backward(dy.float())
    attn_d = attn.cuda()
    rel = lambda a, b_: ((a.float().cpu() - b_).norm() / b_.norm()).item()
    for literal in (True, False):
        mod = ltr.ContextParallelAttention(attn_d, Args, cp_group=ltr.LocalCPGroup(W), literal=literal)
        attn_d.zero_grad()
        xd = x.cuda().requires_grad_(True)
        y = mod(xd, fc.cuda())
        y.backward(dy.cuda())
        assert y.shape == (W, B, Sl, dim)
        assert y.dtype == dtype
        assert (y.detach().cpu().float() - ref.detach()).abs().max() < y_tol
        assert rel(xd.grad, xr.grad) < g_tol
        for n, p_ in attn_d.named_parameters():
            assert rel(p_.grad, ws[n].grad) < g_tol, n
    # passthrough without a cp group (parallel_cp.py:161-162)
    called = {}
    attn_d.forward = lambda x_, f_: called.setdefault("y", x_)
    mod = ltr.ContextParallelAttention(attn_d, Args)
    assert mod(x[0].cuda(), fc.cuda()) is called["y"]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_kernel_bit_exact(ltr, dtype):
    """ltr_rope_apply against the oracle's restatement of apply_rotary_emb (layers/layers.py:44-70): the kernel
    rounds the four products of the complex multiply separately, as torch's fp32 complex multiply on the CPU
    does, so forward and gradient agree bit for bit in fp32 and therefore after the cast to bf16 as well."""
    g = torch.Generator().manual_seed(11)
    for (B, S, H, Hk, D) in ((2, 37, 3, 3, 64), (1, 64, 8, 2, 128), (1, 5, 1, 1, 8)):
        q = torch.randn(B, S, H, D, generator=g).to(dtype)
        k = torch.randn(B, S, Hk, D, generator=g).to(dtype)
        fc = orc.precompute_freqs_cis(D, S + 3)[3:]                 # a chunk that starts at position 3
        rq, _ = orc.apply_rotary_emb(q, q, fc)
        rk, _ = orc.apply_rotary_emb(k, k, fc)
        qd, kd = q.cuda().requires_grad_(True), k.cuda().requires_grad_(True)
        gq, gk = ltr.apply_rotary_emb(qd, kd, fc.cuda())
        assert gq.dtype == dtype and torch.equal(gq.detach().cpu(), rq) and torch.equal(gk.detach().cpu(), rk)
        # gradient = rotation by the conjugate angles; the oracle's comes from torch autograd on the CPU
        dq_ = torch.randn(B, S, H, D, generator=g).to(dtype)
        qc = q.clone().requires_grad_(True)
        orc.apply_rotary_emb(qc, qc, fc)[0].backward(dq_)
        gq.backward(dq_.cuda())
        assert torch.equal(qd.grad.cpu(), qc.grad)
    # strided input: a [B, H, S, D] buffer viewed as [B, S, H, D]
    x = torch.randn(2, 4, 16, 64, generator=g).to(dtype)
    fc = orc.precompute_freqs_cis(64, 16)
    ref, _ = orc.apply_rotary_emb(x.transpose(1, 2), x.transpose(1, 2), fc)
    got, _ = ltr.apply_rotary_emb(x.cuda().transpose(1, 2), x.cuda().transpose(1, 2), fc.cuda())
    assert torch.equal(got.cpu(), ref)
    with pytest.raises(AssertionError):
        ltr.apply_rotary_emb(x.cuda().transpose(1, 2), x.cuda().transpose(1, 2), fc.cuda()[:8])


@pytest.mark.parametrize("D,Hq,Hkv,dtype,causal", [(96, 4, 2, torch.bfloat16, True), (32, 2, 2, torch.bfloat16, False),
                                                     (80, 4, 4, torch.bfloat16, True), (40, 2, 1, torch.float32, True)])
def test_other_head_dims_take_the_padded_path(ltr, D, Hq, Hkv, dtype, causal):
    """Head dims other than 64 / 128 (the reference takes any dim // n_heads, model/model.py:135): block_attention
    zero-pads them to the next instantiated head dim and keeps the scale 1/sqrt(D) of the true one.  Two ragged chunks,
    GQA, forward and all three gradients against the dense oracle; head dims the padded path cannot serve are refused."""
    g = torch.Generator().manual_seed(300 + D)
    B, Sq, lens, starts = 2, 150, [70, 130], [0, 70]
    qp = 50
    q, do = _randn((B, Sq, Hq, D), g, dtype), _randn((B, Sq, Hq, D), g, dtype)
    ks = [_randn((B, n, Hkv, D), g, dtype) for n in lens]
    vs = [_randn((B, n, Hkv, D), g, dtype) for n in lens]
    o_ref, lse_ref, dq_ref, dk_ref, dv_ref = orc.dense_attention_grads(
        q.float(), torch.cat(ks, 1).float(), torch.cat(vs, 1).float(), do.float(), torch.arange(Sq) + qp, torch.arange(200), causal,
        dtype=torch.float32)
    qd = q.cuda().requires_grad_(True)
    kd = [k.cuda().requires_grad_(True) for k in ks]
    vd = [v.cuda().requires_grad_(True) for v in vs]
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")          # the slow path announces itself once per process
        o, lse = ltr.block_attention(qd, kd, vd, starts, qp, None, causal)
    o.backward(do.cuda())
    assert o.shape == (B, Sq, Hq, D)
    f32 = dtype == torch.float32
    assert (o.detach().cpu().float() - o_ref).abs().max() < (F32_TOL if f32 else O_TOL_BF16)
    assert (lse.cpu() - lse_ref).abs().max() < (F32_TOL if f32 else LSE_TOL_BF16)
    tol = 1e-3 if f32 else GRAD_RTOL_BF16
    assert _rel(qd.grad.cpu(), dq_ref) < tol
    assert _rel(torch.cat([k.grad for k in kd], 1).cpu(), dk_ref) < tol
    assert _rel(torch.cat([v.grad for v in vd], 1).cpu(), dv_ref) < tol
    for bad in (136, 100):
        x = torch.zeros(1, 8, 2, bad, dtype=torch.bfloat16, device="cuda")
        with pytest.raises(RuntimeError, match="head dim"):
            ltr.block_attention(x, [x], [x], [0])


@pytest.mark.gpu
def test_attention_layer_gqa(ltr):
    """lightron_amd.Attention (model/model.py:123-202 on the HIP kernels) against the reference composition restated
    with the oracle: projections, RoPE, repeat_kv (kv head = q head // n_rep), dense causal attention, wo; forward
    and the gradients of the input and of every weight."""
    class Args:
        dim, n_heads, n_kv_heads, tp_size = 256, 4, 2, 1
    B, S, D = 2, 96, 64
    torch.manual_seed(3)
    layer = ltr.Attention(Args).to(torch.bfloat16)
    x = ((torch.rand(B, S, Args.dim) * 2 - 1) * 0.5).to(torch.bfloat16)
    dy = ((torch.rand(B, S, Args.dim) * 2 - 1) * 0.1).to(torch.bfloat16)
    fc = orc.precompute_freqs_cis(D, S)
    # oracle in fp32 on the CPU from the same bf16 parameters
    ws = {n: p.detach().float().requires_grad_(True) for n, p in layer.named_parameters()}
    xr = x.float().requires_grad_(True)
    q = (xr @ ws["wq.weight"].T).view(B, S, 4, D)
    k = (xr @ ws["wk.weight"].T).view(B, S, 2, D)
    v = (xr @ ws["wv.weight"].T).view(B, S, 2, D)
    q, k = orc.apply_rotary_emb(q, k, fc)
    assert torch.equal(ltr.repeat_kv(k, 2), k.repeat_interleave(2, dim=2))      # model.py:11-34
    pos = torch.arange(S)
    o, _ = orc.dense_attention(q, k, v, pos, pos, True)
    y_ref = o.float().flatten(2) @ ws["wo.weight"].T
    y_ref.backward(dy.float())
    ld = layer.cuda()
    xd = x.cuda().requires_grad_(True)
    y = ld(xd, fc.cuda())
    y.backward(dy.cuda())
    assert y.shape == (B, S, Args.dim) and y.dtype == torch.bfloat16
    rel = lambda a, b: ((a.float().cpu() - b).norm() / b.norm()).item()
    assert rel(y, y_ref.detach()) < 2e-2
    assert rel(xd.grad, xr.grad) < 5e-2
    for n, p in ld.named_parameters():
        assert rel(p.grad, ws[n].grad) < 5e-2, n
    with pytest.raises(NotImplementedError):
        class A2(Args):
            tp_size = 2
        ltr.Attention(A2)


@pytest.mark.gpu
def test_against_library_sdpa_on_gpu(ltr):
    """Independent of the oracle: the installed torch's scaled_dot_product_attention on the GPU (the routine the
    reference itself calls, model/model.py:193-198) in fp32 on the same bf16 inputs, GQA by repeat_interleave,
    causal; forward and all three gradients at a size the dense oracle would take minutes for."""
    import torch.nn.functional as F
    B, S, Hq, Hkv, D = 2, 2048, 8, 2, 128
    g = torch.Generator().manual_seed(5)
    q, k, v, do = (torch.randn(B, S, h, D, generator=g).to(torch.bfloat16).cuda() for h in (Hq, Hkv, Hkv, Hq))
    qr, kr, vr = (t.float().requires_grad_(True) for t in (q, k, v))
    rep = Hq // Hkv
    o_ref = F.scaled_dot_product_attention(qr.transpose(1, 2), kr.repeat_interleave(rep, 2).transpose(1, 2),
                                           vr.repeat_interleave(rep, 2).transpose(1, 2), is_causal=True).transpose(1, 2)
    o_ref.backward(do.float())
    qd, kd, vd = (t.clone().requires_grad_(True) for t in (q, k, v))
    o, _ = ltr.block_attention(qd, [kd], [vd], [0], 0, None, causal=True)
    o.backward(do)
    assert (o.float() - o_ref).abs().max().item() < 2e-2
    rel = lambda a, b: ((a.float() - b).norm() / b.norm()).item()
    assert rel(qd.grad, qr.grad) < 5e-2 and rel(kd.grad, kr.grad) < 5e-2 and rel(vd.grad, vr.grad) < 5e-2


@pytest.mark.gpu
def test_dq_written_as_bf16_equals_accumulate_then_cast(ltr):
    """LTR_DQ_BF16 (dq receives the bf16 result of a call that holds every KV chunk) against the fp32 accumulator
    path followed by ltr_cast_f32_to_bf16: the same value is rounded once in both, so the bits agree."""
    g = torch.Generator().manual_seed(9)
    B, Sq, Hq, Hkv, D = 1, 300, 4, 2, 128
    q, do = (torch.randn(B, Sq, Hq, D, generator=g).to(torch.bfloat16).cuda() for _ in range(2))
    kf, vf = (torch.randn(B, 300, Hkv, D, generator=g).to(torch.bfloat16).cuda() for _ in range(2))
    ks, vs, pos0 = [kf[:, :200], kf[:, 200:]], [vf[:, :200], vf[:, 200:]], [0, 200]
    o, lse = ltr.attn_fwd(q, ks, vs, pos0, 0, None, True)
    delta = ltr.attn_delta(o, do)
    dkf, dvf = (torch.zeros(kf.shape, dtype=torch.float32, device="cuda") for _ in range(2))
    dks, dvs = [dkf[:, :200], dkf[:, 200:]], [dvf[:, :200], dvf[:, 200:]]
    acc = torch.zeros(q.shape, dtype=torch.float32, device="cuda")
    ltr.attn_bwd_accumulate(q, do, lse, delta, ks, vs, pos0, acc, dks, dvs, 0, None, True, do_dkdv=False)
    direct = torch.full(q.shape, float("nan"), dtype=torch.bfloat16, device="cuda")
    ltr.attn_bwd_accumulate(q, do, lse, delta, ks, vs, pos0, direct, dks, dvs, 0, None, True, do_dkdv=False)
    assert torch.equal(direct, ltr.cast_to_bf16(acc))
    # LTR_DELTA_FROM_O: the dQ kernel computes DELTA from o and leaves it in the workspace for the dK/dV kernel
    ws = torch.full(delta.shape, float("nan"), dtype=torch.float32, device="cuda")
    direct2 = torch.empty_like(direct)
    ltr.attn_bwd_accumulate(q, do, lse, ws, ks, vs, pos0, direct2, dks, dvs, 0, None, True, o=o)
    assert (ws - delta).abs().max().item() < 1e-4 * delta.abs().max().item() + 1e-5
    assert (direct2.float() - direct.float()).abs().max().item() < 2e-2 * direct.float().abs().max().item()
    dk_sep = torch.zeros_like(dkf)
    dv_sep = torch.zeros_like(dvf)
    ltr.attn_bwd_accumulate(q, do, lse, delta, ks, vs, pos0, acc, [dk_sep[:, :200], dk_sep[:, 200:]],
                            [dv_sep[:, :200], dv_sep[:, 200:]], 0, None, True, do_dq=False)
    assert (dkf - dk_sep).abs().max().item() < 1e-3 * dk_sep.abs().max().item()
    assert (dvf - dv_sep).abs().max().item() < 1e-3 * dv_sep.abs().max().item()
    with pytest.raises(RuntimeError):
        ltr.attn_bwd_accumulate(q, do, lse, ws, ks, vs, pos0, direct2, dks, dvs, 0, None, True, do_dq=False, o=o)
    with pytest.raises(RuntimeError):
        ltr.attn_bwd_accumulate(q, do, lse, delta, ks * 20, vs * 20, pos0 * 20, direct, dks * 20, dvs * 20, 0, None, True)


@pytest.mark.gpu
@pytest.mark.parametrize("D,Hq,Hkv,Sq,q0,causal", [(128, 4, 2, 300, 0, True), (64, 2, 2, 100, 150, True),
                                                   (128, 2, 1, 77, 40, False), (64, 4, 1, 256, 1000, True)])
def test_dkdv_written_as_bf16_equals_accumulate_then_cast(ltr, D, Hq, Hkv, Sq, q0, causal):
    """LTR_DKDV_BF16 (dk / dv receive the bf16 results of a call whose q holds every query that sees the keys) against
    the fp32 accumulator path followed by the cast: the same value is rounded once in both, so the bits agree; keys
    that no query sees (whole 128-key blocks of them included) are written as zeros."""
    g = torch.Generator().manual_seed(21)
    B, sks, pos0 = 2, [200, 130, 400], [0, 200, 330]
    q, do = (torch.randn(B, Sq, Hq, D, generator=g).to(torch.bfloat16).cuda() for _ in range(2))
    kf, vf = (torch.randn(B, sum(sks), Hkv, D, generator=g).to(torch.bfloat16).cuda() for _ in range(2))
    offs = [0, 200, 330]
    cut = lambda t: [t[:, o_:o_ + n_] for o_, n_ in zip(offs, sks)]
    ks, vs = cut(kf), cut(vf)
    o, lse = ltr.attn_fwd(q, ks, vs, pos0, q0, None, causal)
    delta = ltr.attn_delta(o, do)
    dq = torch.empty_like(q)
    dkf, dvf = (torch.zeros(kf.shape, dtype=torch.float32, device="cuda") for _ in range(2))
    ltr.attn_bwd_accumulate(q, do, lse, delta, ks, vs, pos0, dq, cut(dkf), cut(dvf), q0, None, causal, do_dq=False)
    dkb, dvb = (torch.full(kf.shape, float("nan"), dtype=torch.bfloat16, device="cuda") for _ in range(2))
    ltr.attn_bwd_accumulate(q, do, lse, delta, ks, vs, pos0, dq, cut(dkb), cut(dvb), q0, None, causal, do_dq=False)
    assert torch.equal(dkb, ltr.cast_to_bf16(dkf))
    assert torch.equal(dvb, ltr.cast_to_bf16(dvf))
    if causal and q0 + Sq <= 330:
        assert dkb[:, 330:].abs().max() == 0 and dvb[:, 330:].abs().max() == 0   # keys after every query
    with pytest.raises(RuntimeError):   # mixed dtypes
        ltr.attn_bwd_accumulate(q, do, lse, delta, ks, vs, pos0, dq, cut(dkb), cut(dvf), q0, None, causal, do_dq=False)


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["huge_positive", "huge_negative", "mixed_rows", "growing"])
def test_extreme_logits(ltr, case):
    """Scores far outside the range where exp2 of (score - fixed reference) is representable: the forward's
    range check on the row sums must move the reference (up on overflow, down when everything would flush) and
    still match the dense fp64 formula; causal, two KV chunks, GQA."""
    g = torch.Generator().manual_seed(13)
    B, S, Hq, Hkv, D = 1, 256, 4, 2, 64
    q = torch.randn(B, S, Hq, D, generator=g)
    k = torch.randn(B, S, Hkv, D, generator=g)
    v = torch.randn(B, S, Hkv, D, generator=g)
    u = torch.randn(D, generator=g)
    u = u / u.norm()
    if case == "huge_positive":        # scores ~ +40^2 / 8 = +200 natural units = +290 in the exp2 domain
        q, k = q + 40 * u, k + 40 * u
    elif case == "huge_negative":      # every score ~ -200: exp2(score) flushes to zero with the initial reference
        q, k = q + 40 * u, k - 40 * u
    elif case == "mixed_rows":         # some rows huge positive, some huge negative, some ordinary
        q[:, 0::3] += 40 * u
        q[:, 1::3] -= 40 * u
        k = k + 40 * u
    else:                              # the row max grows from chunk to chunk by hundreds
        k[:, S // 2:] += 60 * u
        q = q + 20 * u
    q, k, v = (t.to(torch.bfloat16) for t in (q, k, v))
    pos = torch.arange(S)
    o_ref, lse_ref = orc.dense_attention(q.float(), k.float(), v.float(), pos, pos, True)
    ks, vs = [k[:, :128].cuda(), k[:, 128:].cuda()], [v[:, :128].cuda(), v[:, 128:].cuda()]
    for stepwise in (False, True):
        qd = q.cuda().requires_grad_(True)
        o, lse = ltr.block_attention(qd, ks, vs, [0, 128], 0, None, causal=True, stepwise=stepwise)
        assert torch.isfinite(o).all() and torch.isfinite(lse).all()
        assert (o.float().cpu() - o_ref).abs().max() < 3e-2
        # LSE comes from sums of bf16-rounded P: 1e-2 absolute as elsewhere for bf16, plus 1e-3 of its size
        assert ((lse.cpu() - lse_ref).abs() <= 1e-2 + 1e-3 * lse_ref.abs()).all()


@pytest.mark.parametrize("seed", list(range(24)))
def test_random_shapes_sweep(ltr, seed):
    """Seeded sweep over shapes the fixed cases do not hit: ragged Sq across the 256-row block size, 1-4 KV chunks
    of unequal length (slices of one buffer), arbitrary chunk positions, a two-segment query (q_split) or not,
    causal or not, GQA ratios, both head dims; forward and all gradients against the dense oracle with
    explicit positions."""
    import random
    rnd = random.Random(1000 + seed)
    g = torch.Generator().manual_seed(2000 + seed)
    D = rnd.choice([64, 128])
    Hkv = rnd.choice([1, 2])
    Hq = Hkv * rnd.choice([1, 2, 4])
    B = rnd.choice([1, 2])
    Sq = rnd.choice([1, 31, 64, 200, 255, 256, 257, 300, 513, 640])
    n_ch = rnd.randint(1, 4)
    sks = [rnd.choice([1, 17, 64, 100, 128, 191, 256, 330]) for _ in range(n_ch)]
    causal = rnd.random() < 0.7
    # chunk positions: disjoint ranges in random order; query segments placed among them
    starts, p = [], rnd.randint(0, 50)
    for sk in sks:
        starts.append(p)
        p += sk + rnd.randint(0, 40)
    order = list(range(n_ch))
    rnd.shuffle(order)
    q_split = rnd.choice([None, rnd.randint(1, Sq)]) if Sq > 1 else None
    if q_split is None or q_split == Sq:
        q_split, qp = None, rnd.randint(0, p)
        q_pos = torch.arange(qp, qp + Sq)
        q_pos0 = qp
    else:
        a0, a1 = rnd.randint(0, p), rnd.randint(0, p + 200)
        q_pos = torch.cat([torch.arange(a0, a0 + q_split), torch.arange(a1, a1 + Sq - q_split)])
        q_pos0 = (a0, a1)
    q = _randn((B, Sq, Hq, D), g, torch.bfloat16)
    do = _randn((B, Sq, Hq, D), g, torch.bfloat16)
    kbuf = _randn((B, sum(sks), Hkv, D), g, torch.bfloat16)
    vbuf = _randn((B, sum(sks), Hkv, D), g, torch.bfloat16)
    offs = [sum(sks[:i]) for i in range(n_ch)]
    k_pos = torch.cat([torch.arange(starts[i], starts[i] + sks[i]) for i in range(n_ch)])
    o_ref, lse_ref, dq_ref, dk_ref, dv_ref = orc.dense_attention_grads(q.float(), kbuf.float(), vbuf.float(), do.float(),
                                                                         q_pos, k_pos, causal)
    kd, vd = kbuf.cuda().requires_grad_(True), vbuf.cuda().requires_grad_(True)
    qd = q.cuda().requires_grad_(True)
    ks = [kd[:, offs[i]:offs[i] + sks[i]] for i in order]
    vs = [vd[:, offs[i]:offs[i] + sks[i]] for i in order]
    o, lse = ltr.block_attention(qd, ks, vs, [starts[i] for i in order], q_pos0, q_split, causal=causal)
    o.backward(do.cuda())
    seen = torch.isfinite(lse_ref)                       # rows that see at least one key
    assert torch.equal(torch.isfinite(lse.cpu()), seen)
    assert (o.float().cpu() - o_ref.float()).abs().max() < O_TOL_BF16
    assert (lse.cpu()[seen] - lse_ref.float()[seen]).abs().max() < LSE_TOL_BF16 if seen.any() else True
    for got, ref in ((qd.grad, dq_ref), (kd.grad, dk_ref), (vd.grad, dv_ref)):
        if ref.abs().max() > 0:
            assert _rel(got.cpu(), ref) < GRAD_RTOL_BF16
        else:   # e.g. one visible key per row: the exact gradient is 0, the kernels leave rounding noise
            assert got.abs().max() < 1e-3


@pytest.mark.parametrize("seed", list(range(16)))
def test_random_shapes_sweep_fp32_and_stepwise(ltr, seed):
    """The same kind of sweep for the fp32 forward kernel and for the step-wise path (one launch per KV chunk, the
    (O, LSE) merge in the epilogue), forward only; fp32 inputs to 1e-4, bf16 inputs to the bf16 tolerances."""
    import random
    rnd = random.Random(5000 + seed)
    g = torch.Generator().manual_seed(6000 + seed)
    dtype = rnd.choice([torch.float32, torch.bfloat16])
    D = rnd.choice([64, 128])
    Hkv = rnd.choice([1, 2])
    Hq = Hkv * rnd.choice([1, 2])
    B = rnd.choice([1, 2])
    Sq = rnd.choice([1, 63, 64, 65, 130, 256, 300])
    n_ch = rnd.randint(1, 4)
    sks = [rnd.choice([1, 17, 64, 100, 128, 191]) for _ in range(n_ch)]
    causal = rnd.random() < 0.7
    starts, p = [], rnd.randint(0, 30)
    for sk in sks:
        starts.append(p)
        p += sk
    qp = rnd.randint(0, p)
    q_pos = torch.arange(qp, qp + Sq)
    q = _randn((B, Sq, Hq, D), g, dtype)
    kbuf = _randn((B, sum(sks), Hkv, D), g, dtype)
    vbuf = _randn((B, sum(sks), Hkv, D), g, dtype)
    offs = [sum(sks[:i]) for i in range(n_ch)]
    k_pos = torch.cat([torch.arange(starts[i], starts[i] + sks[i]) for i in range(n_ch)])
    o_ref, lse_ref = orc.dense_attention(q.float(), kbuf.float(), vbuf.float(), q_pos, k_pos, causal)
    kd, vd = kbuf.cuda(), vbuf.cuda()
    ks = [kd[:, offs[i]:offs[i] + sks[i]] for i in range(n_ch)]
    vs = [vd[:, offs[i]:offs[i] + sks[i]] for i in range(n_ch)]
    o_tol, l_tol = (F32_TOL, F32_TOL) if dtype == torch.float32 else (O_TOL_BF16, LSE_TOL_BF16)
    seen = torch.isfinite(lse_ref)
    for stepwise in (False, True):
        with torch.no_grad():
            o, lse = ltr.block_attention(q.cuda(), ks, vs, starts, qp, None, causal=causal, stepwise=stepwise)
        assert torch.equal(torch.isfinite(lse.cpu()), seen)
        assert (o.float().cpu() - o_ref.float()).abs().max() < o_tol
        if seen.any():
            assert (lse.cpu()[seen] - lse_ref.float()[seen]).abs().max() < l_tol


@pytest.mark.parametrize("seed", list(range(12)))
def test_ring_sweep_all_ranks_forward_backward(ltr, seed):
    """ring_attention_kernel with a LocalRing for every rank of a random ring (world size, layout, causal or not,
    GQA, step-wise or fused): the ranks' outputs, gathered back to sequence order, against dense attention on the
    whole sequence; dQ per rank and dK/dV summed over the ranks against its gradients."""
    import random
    rnd = random.Random(7000 + seed)
    g = torch.Generator().manual_seed(8000 + seed)
    W = rnd.choice([1, 2, 3, 4, 5])
    layout = rnd.choice(["contiguous", "zigzag"])
    causal = rnd.random() < 0.7
    stepwise = rnd.random() < 0.4
    D = rnd.choice([64, 128])
    Hkv = rnd.choice([1, 2])
    Hq = Hkv * rnd.choice([1, 2, 4])
    B = rnd.choice([1, 2])
    Sl = rnd.choice([2, 34, 64, 96, 130, 256])
    S = W * Sl
    q, do = (_randn((B, S, Hq, D), g, torch.bfloat16) for _ in range(2))
    k, v = (_randn((B, S, Hkv, D), g, torch.bfloat16) for _ in range(2))
    pos = torch.arange(S)
    o_ref, lse_ref, dq_ref, dk_ref, dv_ref = orc.dense_attention_grads(q.float(), k.float(), v.float(), do.float(), pos, pos, causal)
    share = [orc.zigzag_positions(r, W, S) if layout == "zigzag" else orc.contiguous_positions(r, Sl) for r in range(W)]
    kd = [k[:, share[r]].contiguous().cuda().requires_grad_(True) for r in range(W)]
    vd = [v[:, share[r]].contiguous().cuda().requires_grad_(True) for r in range(W)]
    for r in range(W):
        qr = q[:, share[r]].contiguous().cuda().requires_grad_(True)
        ring = ltr.LocalRing(r, W, kv=list(zip(kd, vd)), causal=causal, layout=layout, stepwise=stepwise)
        o = ltr.ring_attention_kernel(qr, kd[r], vd[r], ring, None)
        o.backward(do[:, share[r]].contiguous().cuda())
        assert (o.float().cpu() - o_ref[:, share[r]].float()).abs().max() < O_TOL_BF16
        assert (ring.last_lse.cpu() - lse_ref[:, :, share[r]].float()).abs().max() < LSE_TOL_BF16
        assert _rel(qr.grad.cpu(), dq_ref[:, share[r]]) < GRAD_RTOL_BF16
    # each rank's backward added a bf16-rounded contribution to the chunks' .grad: W roundings instead of one
    dk = torch.zeros_like(dk_ref)
    dv = torch.zeros_like(dv_ref)
    for r in range(W):
        dk[:, share[r]] = kd[r].grad.cpu().double()
        dv[:, share[r]] = vd[r].grad.cpu().double()
    assert _rel(dk, dk_ref) < GRAD_RTOL_BF16 and _rel(dv, dv_ref) < GRAD_RTOL_BF16


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_ring_fp32_kv_grads_one_cast(ltr, seed):
    """RingKVGrads: dK / dV summed over the ranks in fp32 and cast once.  Against the dense gradients, and closer to them
    (or as close) than the sum of per-rank bf16 gradients; nothing reaches k.grad before finalize()."""
    import random
    rnd = random.Random(7100 + seed)
    g = torch.Generator().manual_seed(8100 + seed)
    W, layout = rnd.choice([2, 4, 6]), rnd.choice(["contiguous", "zigzag"])
    D, Hkv, Hq, B, Sl = rnd.choice([64, 128]), 2, 4, rnd.choice([1, 2]), rnd.choice([64, 130, 256])
    S = W * Sl
    q, do = (_randn((B, S, Hq, D), g, torch.bfloat16) for _ in range(2))
    k, v = (_randn((B, S, Hkv, D), g, torch.bfloat16) for _ in range(2))
    pos = torch.arange(S)
    _, _, dq_ref, dk_ref, dv_ref = orc.dense_attention_grads(q.float(), k.float(), v.float(), do.float(), pos, pos, True)
    share = [orc.zigzag_positions(r, W, S) if layout == "zigzag" else orc.contiguous_positions(r, Sl) for r in range(W)]
    errs = {}
    for mode in ("fp32", "bf16"):
        kd = [k[:, share[r]].contiguous().cuda().requires_grad_(True) for r in range(W)]
        vd = [v[:, share[r]].contiguous().cuda().requires_grad_(True) for r in range(W)]
        kv = list(zip(kd, vd))
        grads = ltr.RingKVGrads(kv) if mode == "fp32" else None
        for r in range(W):
            qr = q[:, share[r]].contiguous().cuda().requires_grad_(True)
            ring = ltr.LocalRing(r, W, kv=kv, causal=True, layout=layout, kv_grads=grads)
            ltr.ring_attention_kernel(qr, kd[r], vd[r], ring, None).backward(do[:, share[r]].contiguous().cuda())
            assert _rel(qr.grad.cpu(), dq_ref[:, share[r]]) < GRAD_RTOL_BF16
        if grads is not None:
            assert all(t.grad is None for t in kd + vd)
            grads.finalize()
        dk, dv = torch.zeros_like(dk_ref), torch.zeros_like(dv_ref)
        for r in range(W):
            dk[:, share[r]], dv[:, share[r]] = kd[r].grad.cpu().double(), vd[r].grad.cpu().double()
        errs[mode] = (_rel(dk, dk_ref), _rel(dv, dv_ref))
        assert max(errs[mode]) < GRAD_RTOL_BF16
    assert errs["fp32"][0] <= errs["bf16"][0] * 1.05 and errs["fp32"][1] <= errs["bf16"][1] * 1.05, errs


@pytest.mark.parametrize("dtype,n_chunks", [(torch.bfloat16, 40), (torch.bfloat16, 70), (torch.float32, 35)])
def test_more_chunks_than_one_launch_holds(ltr, dtype, n_chunks):
    """More KV chunks than one launch's table (32): the host splits them into several launches.  Forward: the later
    launches merge into the (O, LSE) of the earlier ones (LTR_MERGE); backward: DELTA from O on the first launch only, dQ
    accumulated in fp32 over the launches and cast, dK / dV of each launch's chunks written by it.  Ragged chunk lengths
    of 16-64 keys, GQA, causal with the chunks' positions shuffled, through block_attention and autograd, against the
    dense oracle."""
    import random
    rnd = random.Random(4200 + n_chunks)
    g = torch.Generator().manual_seed(4300 + n_chunks)
    B, Hq, Hkv, D = 2, 4, 2, 128 if dtype == torch.bfloat16 else 64
    lens = [rnd.randint(16, 64) for _ in range(n_chunks)]
    starts = [sum(lens[:i]) for i in range(n_chunks)]
    Sk = sum(lens)
    Sq = 200
    q_pos0 = Sk - Sq - 37                                # the last keys are invisible to every query
    q, do = (_randn((B, Sq, Hq, D), g, dtype) for _ in range(2))
    k, v = (_randn((B, Sk, Hkv, D), g, dtype) for _ in range(2))
    o_ref, lse_ref, dq_ref, dk_ref, dv_ref = orc.dense_attention_grads(
        q.float(), k.float(), v.float(), do.float(), torch.arange(Sq) + q_pos0, torch.arange(Sk), True)
    order = list(range(n_chunks))
    rnd.shuffle(order)                                   # visiting order != position order
    qd = q.cuda().requires_grad_(True)
    kl = [k[:, starts[j]:starts[j] + lens[j]].contiguous().cuda().requires_grad_(True) for j in order]
    vl = [v[:, starts[j]:starts[j] + lens[j]].contiguous().cuda().requires_grad_(True) for j in order]
    o, lse = ltr.block_attention(qd, kl, vl, [starts[j] for j in order], q_pos0, None, True)
    o.backward(do.cuda())
    f32 = dtype == torch.float32
    assert (o.detach().cpu().double() - o_ref).abs().max() < (F32_TOL if f32 else O_TOL_BF16)
    assert (lse.cpu().double() - lse_ref).abs().max() < (F32_TOL if f32 else LSE_TOL_BF16)
    dk, dv = torch.zeros_like(dk_ref), torch.zeros_like(dv_ref)
    for i, j in enumerate(order):
        dk[:, starts[j]:starts[j] + lens[j]] = kl[i].grad.cpu().double()
        dv[:, starts[j]:starts[j] + lens[j]] = vl[i].grad.cpu().double()
    if f32:
        assert (qd.grad.cpu().double() - dq_ref).abs().max() < F32_TOL * max(1.0, dq_ref.abs().max().item())
        assert (dk - dk_ref).abs().max() < F32_TOL * max(1.0, dk_ref.abs().max().item())
        assert (dv - dv_ref).abs().max() < F32_TOL * max(1.0, dv_ref.abs().max().item())
    else:
        assert _rel(qd.grad.cpu(), dq_ref) < GRAD_RTOL_BF16
        assert _rel(dk, dk_ref) < GRAD_RTOL_BF16 and _rel(dv, dv_ref) < GRAD_RTOL_BF16
    assert dk[:, q_pos0 + Sq:].abs().max() == 0 and dv[:, q_pos0 + Sq:].abs().max() == 0    # keys no query sees


@pytest.mark.parametrize("D,Hq,Hkv,Sq,q_pos,chunks,causal", [
    (128, 4, 2, 300, (1000, 1000), [(700, 400), (1100, 200)], True),      # contiguous rows, two KV chunks
    (64, 4, 4, 256, (0, 768), [(0, 512), (512, 512)], True),              # zig-zag rows (two segments), D = 64
    (128, 2, 1, 77, (130000, 130000), [(129900, 250)], False),            # positions near the top of a 131072 table
])
def test_fused_rope_prologue_and_dq_epilogue(ltr, D, Hq, Hkv, Sq, q_pos, chunks, causal):
    """LTR_ROPE_Q / LTR_ROPE_DQ against the separate pass (ltr_rope_apply on q, attention, conjugate ltr_rope_apply on
    dQ) and against the oracle (apply_rotary_emb restated, then dense attention and its autograd).  The rotated q and
    therefore O and LSE must have the SAME BITS as with the separate pass; dQ is rounded once instead of twice, so it is
    compared with a tolerance (and must not be further from the oracle than the two-pass result)."""
    g = torch.Generator().manual_seed(31 + Sq)
    B = 2
    n_pos = max(max(p0 + n for p0, n in chunks), max(q_pos) + Sq) + 5
    fc = orc.precompute_freqs_cis(D, n_pos)
    split = Sq // 2 if q_pos[0] != q_pos[1] else Sq
    qpos = torch.cat([torch.arange(split) + q_pos[0], torch.arange(Sq - split) + q_pos[1]])
    q, do = _randn((B, Sq, Hq, D), g, torch.bfloat16), _randn((B, Sq, Hq, D), g, torch.bfloat16)
    ks = [_randn((B, n, Hkv, D), g, torch.bfloat16) for _, n in chunks]
    vs = [_randn((B, n, Hkv, D), g, torch.bfloat16) for _, n in chunks]
    kpos = torch.cat([torch.arange(n) + p0 for p0, n in chunks])
    # oracle: rotate (fp32 complex multiply, cast back to bf16 as the reference does), dense attention, autograd
    q_rot_ref, _ = orc.apply_rotary_emb(q, q, fc[qpos])
    k_rot = [orc.apply_rotary_emb(k, k, fc[p0:p0 + n])[0] for k, (p0, n) in zip(ks, chunks)]
    o_ref, lse_ref, dq_rot_ref, _, _ = orc.dense_attention_grads(q_rot_ref.float(), torch.cat(k_rot, 1).float(), torch.cat(vs, 1).float(),
                                                                 do.float(), qpos, kpos, causal)
    conj = torch.conj(fc[qpos])
    dq_ref = torch.view_as_real(torch.view_as_complex(dq_rot_ref.float().reshape(B, Sq, Hq, D // 2, 2)) * conj[None, :, None, :]).flatten(3)

    fcd = fc.cuda()
    table = ltr.rope_table(fcd)
    kd = [ltr.rope_one(k.cuda(), fcd[p0:p0 + n]) for k, (p0, n) in zip(ks, chunks)]
    for a, b in zip(kd, k_rot):
        assert torch.equal(a.cpu(), b)
    vd = [v.cuda() for v in vs]
    pos0 = [p0 for p0, _ in chunks]
    qd = q.cuda()
    # separate pass
    q_rot_2p = ltr.rope_one(qd, fcd[qpos.cuda()])
    assert torch.equal(q_rot_2p.cpu(), q_rot_ref)
    o2, lse2 = ltr.attn_fwd(q_rot_2p, kd, vd, pos0, q_pos, split, causal)
    # fused prologue
    q_rot = torch.full_like(qd, float("nan"))
    o1, lse1 = ltr.attn_fwd(qd, kd, vd, pos0, q_pos, split, causal, q_rope=table, q_rot_out=q_rot)
    assert torch.equal(q_rot, q_rot_2p)
    assert torch.equal(o1, o2) and torch.equal(lse1, lse2)
    assert (o1.cpu().double() - o_ref).abs().max() < O_TOL_BF16
    fin = torch.isfinite(lse_ref)
    assert (lse1.cpu().double()[fin] - lse_ref[fin]).abs().max() < LSE_TOL_BF16

    # through autograd: fused (q un-rotated in, gradient of un-rotated q out) and two-pass
    def grads(fused):
        qg = qd.clone().requires_grad_(True)
        if fused:
            o, _ = ltr.block_attention(qg, kd, vd, pos0, q_pos, split, causal, q_rope=table)
        else:
            o, _ = ltr.block_attention(ltr.rope_one(qg, fcd[qpos.cuda()]), kd, vd, pos0, q_pos, split, causal)
        o.backward(do.cuda())
        return qg.grad.cpu()
    dq_f, dq_2 = grads(True), grads(False)
    e_f, e_2 = _rel(dq_f, dq_ref), _rel(dq_2, dq_ref)
    assert e_f < GRAD_RTOL_BF16 and e_2 < GRAD_RTOL_BF16, (e_f, e_2)
    assert e_f <= e_2 * 1.05 + 1e-4, (e_f, e_2)                     # one rounding instead of two
    assert _rel(dq_f, dq_2.double()) < 1e-2
    # the fp32 accumulator form of the dQ epilogue (two launches' worth of chunks accumulate rotated partials)
    delta = ltr.attn_delta(o1, do.cuda())
    acc = torch.zeros(qd.shape, dtype=torch.float32, device="cuda")
    dk = [torch.zeros(k.shape, dtype=torch.float32, device="cuda") for k in kd]
    dv = [torch.zeros(k.shape, dtype=torch.float32, device="cuda") for k in kd]
    for i in range(len(kd)):
        ltr.attn_bwd_accumulate(q_rot, do.cuda(), lse1, delta, kd[i:i + 1], vd[i:i + 1], pos0[i:i + 1], acc, dk[i:i + 1], dv[i:i + 1],
                                q_pos, split, causal, do_dkdv=False, dq_rope=table)
    assert _rel(acc.cpu(), dq_ref) < GRAD_RTOL_BF16


@pytest.mark.parametrize("D,B,Hq,Hkv,Sq,q_pos,split,chunks", [
    (128, 8, 32, 32, 700, (0, 0), None, [(0, 700)]),                       # 3 q tiles: a pair and the middle tile alone
    (64, 8, 32, 8, 1100, (300, 300), None, [(0, 1000), (1000, 400)]),      # 5 q tiles, ragged, GQA, two chunks
    (128, 4, 64, 16, 1024, (0, 3072), 512, [(0, 512), (512, 2560), (3072, 512)]),   # zig-zag rows: two segments
])
def test_paired_q_tiles_forward_backward(ltr, D, B, Hq, Hkv, Sq, q_pos, split, chunks):
    """Enough (batch, head) pairs that the host hands the forward and dQ kernels a late q tile and its early counterpart
    per block (q_tile_slots: causal, and the equal blocks fill the 256 CUs evenly).  Odd tile counts (the middle tile runs
    alone), a ragged last tile, GQA, both head dims, two-segment rows; against the dense oracle."""
    g = torch.Generator().manual_seed(77 + Sq)
    # the library itself says whether it pairs the tiles of this launch (for the device this test runs on)
    plan = ltr.attn_plan(B, Hq, Hkv, D, Sq, [n for _, n in chunks], [p0 for p0, _ in chunks], q_pos, split, True)
    n_qt = (Sq + 255) // 256
    assert plan["fwd"]["rows"] == plan["dq"]["rows"] == 256
    assert plan["fwd"]["paired"] and plan["dq"]["paired"], "shape does not trigger the pairing on this device"
    assert plan["fwd"]["blocks"] == plan["dq"]["blocks"] == ((n_qt + 1) // 2) * B * Hq
    sp = Sq if split is None else split
    qpos = torch.cat([torch.arange(sp) + q_pos[0], torch.arange(Sq - sp) + q_pos[1]])
    q, do = _randn((B, Sq, Hq, D), g, torch.bfloat16), _randn((B, Sq, Hq, D), g, torch.bfloat16)
    ks = [_randn((B, n, Hkv, D), g, torch.bfloat16) for _, n in chunks]
    vs = [_randn((B, n, Hkv, D), g, torch.bfloat16) for _, n in chunks]
    kpos = torch.cat([torch.arange(n) + p0 for p0, n in chunks])
    o_ref, lse_ref, dq_ref, dk_ref, dv_ref = orc.dense_attention_grads(q.float(), torch.cat(ks, 1).float(), torch.cat(vs, 1).float(),
                                                                       do.float(), qpos, kpos, True, dtype=torch.float32)
    qd = q.cuda().requires_grad_(True)
    kd = [k.cuda().requires_grad_(True) for k in ks]
    vd = [v.cuda().requires_grad_(True) for v in vs]
    o, lse = ltr.block_attention(qd, kd, vd, [p0 for p0, _ in chunks], q_pos, split, True)
    o.backward(do.cuda())
    assert (o.detach().cpu().float() - o_ref).abs().max() < O_TOL_BF16
    fin = torch.isfinite(lse_ref)
    assert torch.equal(torch.isfinite(lse.cpu()), fin)
    assert (lse.cpu()[fin] - lse_ref[fin]).abs().max() < LSE_TOL_BF16
    assert _rel(qd.grad.cpu(), dq_ref) < GRAD_RTOL_BF16
    assert _rel(torch.cat([k.grad for k in kd], 1).cpu(), dk_ref) < GRAD_RTOL_BF16
    assert _rel(torch.cat([v.grad for v in vd], 1).cpu(), dv_ref) < GRAD_RTOL_BF16


@pytest.mark.parametrize("seed", list(range(8)))
def test_rope_sweep_bit_exact(ltr, seed):
    """ltr_rope_apply on random shapes, dtypes, layouts and starting positions against the oracle, bit for bit."""
    import random
    rnd = random.Random(9000 + seed)
    g = torch.Generator().manual_seed(9100 + seed)
    dtype = rnd.choice([torch.float32, torch.bfloat16])
    B, S, H = rnd.choice([1, 2, 3]), rnd.choice([1, 7, 64, 129]), rnd.choice([1, 2, 5])
    D = rnd.choice([8, 16, 64, 96, 128])
    p0 = rnd.choice([0, 5, 1000, 100000])
    x = _randn((B, H, S, D), g, dtype) if rnd.random() < 0.5 else _randn((B, S, H, D), g, dtype).transpose(1, 2)
    xv = x.transpose(1, 2)                                    # [B, S, H, D] view, one of the two memory layouts
    fc = orc.precompute_freqs_cis(D, p0 + S)[p0:]
    ref, _ = orc.apply_rotary_emb(xv, xv, fc)
    got, _ = ltr.apply_rotary_emb(xv.cuda(), xv.cuda(), fc.cuda())
    assert got.dtype == dtype and torch.equal(got.cpu(), ref)


@pytest.mark.parametrize("seed", list(range(24)))
def test_dkdv_block_size_hints_d64(ltr, seed):
    """Head dim 64: the dK/dV kernel with 128 and with 256 keys per block (LTR_DKDV_KEYS_128 / _256, the latter two 32-key
    halves per wave), forced through the hint flags on shapes that the library's own choice would not send to the wide
    kernel: ragged chunks that end inside a 256-key block, several chunks, GQA, causal with a two-segment query, fp32
    accumulators and bf16 results.  Both against the dense oracle, and against each other to rounding."""
    import random
    rnd = random.Random(7000 + seed)
    g = torch.Generator().manual_seed(8000 + seed)
    D = 64
    Hkv = rnd.choice([1, 2])
    Hq = Hkv * rnd.choice([1, 2, 4])
    B = rnd.choice([1, 2])
    Sq = rnd.choice([64, 100, 256, 300, 513, 700])
    n_ch = rnd.randint(1, 3)
    sks = [rnd.choice([1, 33, 100, 128, 191, 256, 257, 330, 512, 600]) for _ in range(n_ch)]
    causal = rnd.random() < 0.6
    direct = rnd.random() < 0.5          # bf16 results instead of fp32 accumulators
    starts, p = [], rnd.randint(0, 30)
    for sk in sks:
        starts.append(p)
        p += sk + rnd.randint(0, 20)
    q_split = rnd.choice([None, rnd.randint(1, Sq - 1)])
    if q_split is None:
        qp = rnd.randint(0, p)
        q_pos, q_pos0 = torch.arange(qp, qp + Sq), qp
    else:
        a0, a1 = rnd.randint(0, p), rnd.randint(0, p + 100)
        q_pos = torch.cat([torch.arange(a0, a0 + q_split), torch.arange(a1, a1 + Sq - q_split)])
        q_pos0 = (a0, a1)
    q = _randn((B, Sq, Hq, D), g, torch.bfloat16)
    do = _randn((B, Sq, Hq, D), g, torch.bfloat16)
    kbuf = _randn((B, sum(sks), Hkv, D), g, torch.bfloat16)
    vbuf = _randn((B, sum(sks), Hkv, D), g, torch.bfloat16)
    offs = [sum(sks[:i]) for i in range(n_ch)]
    k_pos = torch.cat([torch.arange(starts[i], starts[i] + sks[i]) for i in range(n_ch)])
    _, _, dq_ref, dk_ref, dv_ref = orc.dense_attention_grads(q.float(), kbuf.float(), vbuf.float(), do.float(), q_pos, k_pos, causal)
    qd, dod, kd, vd = _dev(q, do, kbuf, vbuf)
    ks = [kd[:, offs[i]:offs[i] + sks[i]] for i in range(n_ch)]
    vs = [vd[:, offs[i]:offs[i] + sks[i]] for i in range(n_ch)]
    o, lse = ltr.attn_fwd(qd, ks, vs, starts, q_pos0, q_split, causal)
    delta = ltr.attn_delta(o, dod)
    got = {}
    for keys in (128, 256):
        dt = torch.bfloat16 if direct else torch.float32
        dkb = torch.full(kbuf.shape, 7.0 if direct else 0.0, dtype=dt, device="cuda")   # results overwrite, accumulators add
        dvb = torch.full(vbuf.shape, 7.0 if direct else 0.0, dtype=dt, device="cuda")
        dks = [dkb[:, offs[i]:offs[i] + sks[i]] for i in range(n_ch)]
        dvs = [dvb[:, offs[i]:offs[i] + sks[i]] for i in range(n_ch)]
        dq = torch.zeros(q.shape, dtype=torch.float32, device="cuda")
        ltr.attn_bwd_accumulate(qd, dod, lse, delta, ks, vs, starts, dq, dks, dvs, q_pos0, q_split, causal, do_dq=False,
                                dkdv_keys=keys)
        got[keys] = (dkb.float().cpu(), dvb.float().cpu())
        for x, ref in ((got[keys][0], dk_ref), (got[keys][1], dv_ref)):
            if ref.abs().max() > 0:
                assert _rel(x, ref) < GRAD_RTOL_BF16, (keys, seed)
            else:
                assert x.abs().max() < 1e-3
    for a, b_ in zip(got[128], got[256]):
        assert (a - b_).abs().max() <= 2e-2 * max(1.0, b_.abs().max().item())
    # the dQ kernel with 256 and with 512 query rows per block (LTR_DQ_ROWS_256 / _512: two 32-row blocks per wave), fp32
    # accumulator or bf16 result, DELTA given or computed from O by the kernel
    gq = {}
    for rows in (256, 512):
        dq = (torch.full(q.shape, 7.0, dtype=torch.bfloat16, device="cuda") if direct
              else torch.zeros(q.shape, dtype=torch.float32, device="cuda"))
        dlt = torch.full_like(delta, float("nan")) if direct else delta
        ltr.attn_bwd_accumulate(qd, dod, lse, dlt, ks, vs, starts, dq, ks, vs, q_pos0, q_split, causal, do_dkdv=False,
                                o=o if direct else None, dq_rows=rows)
        gq[rows] = dq.float().cpu()
        if direct:
            assert torch.allclose(dlt, delta, rtol=1e-5, atol=1e-5)
        if dq_ref.abs().max() > 0:
            assert _rel(gq[rows], dq_ref) < GRAD_RTOL_BF16, (rows, seed)
        else:
            assert gq[rows].abs().max() < 1e-3
    assert (gq[256] - gq[512]).abs().max() <= 2e-2 * max(1.0, gq[512].abs().max().item())


def test_dkdv_keys_256_refused_where_it_does_not_exist(ltr):
    g = torch.Generator().manual_seed(1)
    q, k, v, do = (_randn((1, 64, 2, 128), g, torch.bfloat16).cuda() for _ in range(4))
    o, lse = ltr.attn_fwd(q, [k], [v], [0])
    delta = ltr.attn_delta(o, do)
    dq = torch.zeros(q.shape, dtype=torch.float32, device="cuda")
    dk, dv = torch.zeros_like(dq), torch.zeros_like(dq)
    with pytest.raises(RuntimeError):
        ltr.attn_bwd_accumulate(q, do, lse, delta, [k], [v], [0], dq, [dk], [dv], dkdv_keys=256)
    with pytest.raises(RuntimeError):
        ltr.attn_bwd_accumulate(q, do, lse, delta, [k], [v], [0], dq, [dk], [dv], dkdv_keys=64)
    with pytest.raises(RuntimeError):
        ltr.attn_bwd_accumulate(q, do, lse, delta, [k], [v], [0], dq, [dk], [dv], dq_rows=512)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_no_query_rows(ltr, dtype):
    """A rank whose q chunk is empty (the reference's matmuls return an empty result there, ring_attention.py:66-104):
    empty O and LSE, zero gradients for K and V, no kernel launch and no error."""
    g = torch.Generator().manual_seed(5)
    q = torch.zeros(2, 0, 4, 64, dtype=dtype).cuda().requires_grad_(True)
    k, v = _dev(_randn((2, 48, 2, 64), g, dtype), _randn((2, 48, 2, 64), g, dtype))
    k.requires_grad_(True)
    v.requires_grad_(True)
    o, lse = ltr.block_attention(q, [k], [v], [0], 0, None, True)
    assert tuple(o.shape) == (2, 0, 4, 64) and tuple(lse.shape) == (2, 4, 0) and o.dtype == dtype
    o.sum().backward()
    torch.cuda.synchronize()
    assert tuple(q.grad.shape) == (2, 0, 4, 64)
    assert k.grad is not None and v.grad is not None
    assert float(k.grad.float().abs().max()) == 0.0 and float(v.grad.float().abs().max()) == 0.0
    # the low-level calls as well
    o2, lse2 = ltr.attn_fwd(q.detach(), [k.detach()], [v.detach()], [0])
    assert o2.numel() == 0 and lse2.numel() == 0
    assert ltr.attn_delta(o2, o2).numel() == 0


@pytest.mark.parametrize("seed", list(range(24)))
def test_fwd_block_size_hints_d64(ltr, seed):
    """Head dim 64: the forward kernel with 256 and with 512 query rows per block (LTR_FWD_ROWS_256 / _512, the latter two
    32-row blocks per wave and 64-key tiles), forced through the hint flags: ragged rows and chunks, several chunks, GQA,
    causal with a two-segment query (so that the paired and the unpaired hand-out of q tiles both occur), bf16 and fp32
    output, one launch or a stepwise merge, optionally with the fused RoPE prologue.  Both against the dense oracle and
    against each other to rounding; the rotated q must have the same bits."""
    import random
    rnd = random.Random(9000 + seed)
    g = torch.Generator().manual_seed(9500 + seed)
    D = 64
    Hkv = rnd.choice([1, 2])
    Hq = Hkv * rnd.choice([1, 2, 4])
    B = rnd.choice([1, 2])
    Sq = rnd.choice([31, 64, 300, 512, 513, 700, 1024, 1300])
    n_ch = rnd.randint(1, 3)
    sks = [rnd.choice([1, 33, 64, 100, 128, 191, 257, 330, 600]) for _ in range(n_ch)]
    causal = rnd.random() < 0.6
    out_dtype = rnd.choice([torch.bfloat16, torch.float32])
    stepwise = n_ch > 1 and rnd.random() < 0.5
    rope = rnd.random() < 0.4
    starts, p = [], rnd.randint(0, 30)
    for sk in sks:
        starts.append(p)
        p += sk + rnd.randint(0, 20)
    q_split = rnd.choice([None, rnd.randint(1, Sq - 1)])
    if q_split is None:
        qp = rnd.randint(0, p + 400)
        q_pos, q_pos0 = torch.arange(qp, qp + Sq), qp
    else:
        a0, a1 = rnd.randint(0, p), rnd.randint(0, p + 400)
        q_pos = torch.cat([torch.arange(a0, a0 + q_split), torch.arange(a1, a1 + Sq - q_split)])
        q_pos0 = (a0, a1)
    q = _randn((B, Sq, Hq, D), g, torch.bfloat16)
    kbuf = _randn((B, sum(sks), Hkv, D), g, torch.bfloat16)
    vbuf = _randn((B, sum(sks), Hkv, D), g, torch.bfloat16)
    offs = [sum(sks[:i]) for i in range(n_ch)]
    k_pos = torch.cat([torch.arange(starts[i], starts[i] + sks[i]) for i in range(n_ch)])
    table, q_in = None, q
    if rope:
        fc = orc.precompute_freqs_cis(D, int(q_pos.max()) + 2)
        q_in, _ = orc.apply_rotary_emb(q, q, fc[q_pos])          # what the kernel's prologue must produce
        table = ltr.rope_table(fc.cuda())
    o_ref, lse_ref = orc.dense_attention(q_in.float(), kbuf.float(), vbuf.float(), q_pos, k_pos, causal)
    qd, kd, vd = _dev(q, kbuf, vbuf)
    ks = [kd[:, offs[i]:offs[i] + sks[i]] for i in range(n_ch)]
    vs = [vd[:, offs[i]:offs[i] + sks[i]] for i in range(n_ch)]
    got = {}
    for rows in (256, 512):
        q_rot = torch.full_like(qd, float("nan")) if rope else None
        if stepwise:
            o, lse = ltr.attn_fwd(qd, ks[:1], vs[:1], starts[:1], q_pos0, q_split, causal, out_dtype=torch.float32,
                                  q_rope=table, q_rot_out=q_rot, fwd_rows=rows)
            for i in range(1, n_ch):
                ltr.attn_fwd(qd, ks[i:i + 1], vs[i:i + 1], starts[i:i + 1], q_pos0, q_split, causal, out=o, lse=lse, merge=True,
                             q_rope=table, fwd_rows=rows)
        else:
            o, lse = ltr.attn_fwd(qd, ks, vs, starts, q_pos0, q_split, causal, out_dtype=out_dtype, q_rope=table,
                                  q_rot_out=q_rot, fwd_rows=rows)
        if rope:
            assert torch.equal(q_rot.cpu(), q_in), (rows, seed)
        got[rows] = (o.float().cpu(), lse.cpu())
        assert (got[rows][0].double() - o_ref).abs().max() < O_TOL_BF16, (rows, seed)
        fin = torch.isfinite(lse_ref)
        assert (got[rows][1].double()[fin] - lse_ref[fin]).abs().max() < LSE_TOL_BF16, (rows, seed)
        assert torch.isinf(got[rows][1][~fin]).all()
    assert (got[256][0] - got[512][0]).abs().max() <= 2e-2
    fin = torch.isfinite(got[256][1])
    assert torch.equal(fin, torch.isfinite(got[512][1]))
    assert (got[256][1][fin] - got[512][1][fin]).abs().max() <= 1e-3


def test_fwd_rows_512_refused_where_it_does_not_exist(ltr):
    g = torch.Generator().manual_seed(2)
    q, k, v = (_randn((1, 64, 2, 128), g, torch.bfloat16).cuda() for _ in range(3))
    with pytest.raises(RuntimeError):
        ltr.attn_fwd(q, [k], [v], [0], fwd_rows=512)            # head dim 128
    with pytest.raises(RuntimeError):
        ltr.attn_fwd(q, [k], [v], [0], fwd_rows=128)
    q, k, v = (_randn((1, 64, 2, 64), g, torch.float32).cuda() for _ in range(3))
    with pytest.raises(RuntimeError):
        ltr.attn_fwd(q, [k], [v], [0], fwd_rows=512)            # fp32
