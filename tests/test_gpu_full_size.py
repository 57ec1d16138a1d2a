"""Full-size GPU tests of the benchmark configs 2-5.  The dense oracle does not finish in seconds at
these sizes, so each test checks sampled query rows (O, LSE, dQ) and sampled keys (dK, dV)
against the oracle's closed form restricted to those rows / keys (fp64, CPU, same seeded bf16
inputs), plus size-independent identities: sum_j dV_j = sum_i dO_i per kv group (softmax rows
sum to one), and step-wise merge == fused launch."""
import pytest
import torch

from oracle import ring_attention_oracle as orc

pytestmark = pytest.mark.gpu

O_TOL, LSE_TOL, GRAD_RTOL = 2e-2, 2e-2, 5e-2


def _rel(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-30)).item()


def _edges(marks, size, n_b, n_h):
    """Deterministic samples on both sides of the boundaries in `marks` (tile, half-chunk and segment edges):
    indices m - 1 and m for every mark inside (0, size), batches and heads taken in turn."""
    idx = sorted({i for m in marks for i in (m - 1, m) if 0 <= i < size})
    return [(j % n_b, (3 * j + 1) % n_h, i) for j, i in enumerate(idx)]


def _check_rows(q, k, v, qpos, kpos, causal, o, lse, do=None, dq=None, n=24, seed=0, edge_rows=()):
    g = torch.Generator().manual_seed(seed)
    B, Sq, Hq, _ = q.shape
    rows = [(int(torch.randint(B, (1,), generator=g)), int(torch.randint(Hq, (1,), generator=g)),
             int(torch.randint(Sq, (1,), generator=g))) for _ in range(n)]
    rows += [(0, 0, 0), (B - 1, Hq - 1, Sq - 1)]
    # block edges of the kernels (256-row q tiles: rows 255 / 256) and the caller's own edges (segment split, ragged end)
    rows += _edges([256, Sq] + list(edge_rows), Sq, B, Hq)
    ref = orc.sampled_rows(q, k, v, qpos, kpos, causal, rows, do)
    num = den = 0.0
    for (b, h, i), (ro, rl, rdq) in zip(rows, ref):
        assert (o[b, i, h].double() - ro).abs().max() < O_TOL, ("O", b, h, i)
        assert abs(lse[b, h, i].double() - rl) < LSE_TOL, ("LSE", b, h, i)
        if dq is not None:
            num += (dq[b, i, h].double() - rdq).pow(2).sum().item()
            den += rdq.pow(2).sum().item()
    if dq is not None:
        assert (num / den) ** 0.5 < GRAD_RTOL, ("dQ", (num / den) ** 0.5)


def _check_keys(q, k, v, o, lse, do, qpos, kpos, causal, dk, dv, n=6, seed=1, edge_keys=()):
    g = torch.Generator().manual_seed(seed)
    B, Sk, Hkv, _ = k.shape
    keys = [(int(torch.randint(B, (1,), generator=g)), int(torch.randint(Hkv, (1,), generator=g)),
             int(torch.randint(Sk, (1,), generator=g))) for _ in range(n)]
    keys += [(0, 0, 0), (B - 1, Hkv - 1, Sk - 1)]
    # block edges of the dK/dV kernel (128-key blocks: keys 127 / 128) and the caller's own (chunk and half-chunk boundaries,
    # the last tile a diagonal sees)
    keys += _edges([128] + list(edge_keys), Sk, B, Hkv)
    ref = orc.sampled_keys(q, k, v, o, lse, do, qpos, kpos, causal, keys)
    nk = dk_ = nv = dv_ = 0.0
    for (b, gi, j), (rk, rv) in zip(keys, ref):
        nk += (dk[b, j, gi].double() - rk).pow(2).sum().item()
        dk_ += rk.pow(2).sum().item()
        nv += (dv[b, j, gi].double() - rv).pow(2).sum().item()
        dv_ += rv.pow(2).sum().item()
    assert (nk / dk_) ** 0.5 < GRAD_RTOL and (nv / dv_) ** 0.5 < GRAD_RTOL, ((nk / dk_) ** 0.5, (nv / dv_) ** 0.5)


def test_config2_full(ltr):
    """B=4, Hq=Hkv=32, D=128, bf16, causal; rank 7's Q chunk of 1024 against 8 KV chunks of 1024;
    q, k, v ~ N(0,1)*0.5, seed 0; fused launch and step-wise launches with the merge epilogue."""
    g = torch.Generator().manual_seed(0)
    B, H, D, sl, W = 4, 32, 128, 1024, 8
    mk = lambda *s: (torch.randn(s, generator=g) * 0.5).to(torch.bfloat16)
    q, k, v = mk(B, sl, H, D), mk(B, W * sl, H, D), mk(B, W * sl, H, D)
    kd, vd = k.cuda(), v.cuda()
    kv = [(kd[:, j * sl:(j + 1) * sl], vd[:, j * sl:(j + 1) * sl]) for j in range(W)]
    qpos, kpos = torch.arange(sl) + 7 * sl, torch.arange(W * sl)
    outs = []
    for stepwise in (False, True):
        ring = ltr.LocalRing(7, W, kv, causal=True, stepwise=stepwise)
        o = ltr.ring_attention_kernel(q.cuda(), kv[7][0], kv[7][1], ring, None)
        _check_rows(q, k, v, qpos, kpos, True, o.cpu(), ring.last_lse.cpu(), n=16)
        outs.append((o, ring.last_lse))
    assert (outs[0][0].float() - outs[1][0].float()).abs().max() < 1e-2
    assert (outs[0][1] - outs[1][1]).abs().max() < 1e-3     # l sums bf16-rounded P: order-dependent rounding


@pytest.mark.parametrize("path", ["accumulators", "bench"])
def test_config3_full_all_ranks(ltr, path):
    """B=1, Hq=32, Hkv=8, D=128, S=32768 as 8 zig-zag rank shares, bf16, causal, N(0,1) seed 0:
    O, LSE, dQ, dK, dV of the whole sequence.  path "accumulators": separate DELTA launch, fp32 dQ accumulator, one
    backward call; path "bench": exactly the call sequence bench.py times - a dQ-only call that computes DELTA from O
    into a shared workspace and writes bf16 dQ (LTR_DELTA_FROM_O | LTR_DQ_BF16), then a dK/dV-only call that reads
    that workspace."""
    g = torch.Generator().manual_seed(0)
    B, Hq, Hkv, D, S, W = 1, 32, 8, 128, 32768, 8
    mk = lambda h: torch.randn(B, S, h, D, generator=g).to(torch.bfloat16)
    q, k, v, do = mk(Hq), mk(Hkv), mk(Hkv), mk(Hq)
    rp = [orc.zigzag_positions(r, W, S) for r in range(W)]
    qd, kd, vd, dod = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    sl, hc = S // W, S // (2 * W)
    ksh = [kd[:, p.cuda()].contiguous() for p in rp]
    vsh = [vd[:, p.cuda()].contiguous() for p in rp]
    dk_acc = [torch.zeros(x.shape, dtype=torch.float32, device="cuda") for x in ksh]
    dv_acc = [torch.zeros(x.shape, dtype=torch.float32, device="cuda") for x in vsh]
    o = torch.empty_like(qd)
    lse = torch.empty(B, Hq, S, device="cuda")
    dq = torch.empty(qd.shape, dtype=torch.float32, device="cuda")
    delta_ws = torch.empty(B, Hq, sl, dtype=torch.float32, device="cuda")       # one workspace for all shares, as in bench.py
    for r in range(W):
        idx = rp[r].cuda()
        ql, dol = qd[:, idx].contiguous(), dod[:, idx].contiguous()
        ks, vs, dks, dvs, pos = [], [], [], [], []
        for j in orc.ring_order(r, W):
            ks += [ksh[j][:, :hc], ksh[j][:, hc:]]
            vs += [vsh[j][:, :hc], vsh[j][:, hc:]]
            dks += [dk_acc[j][:, :hc], dk_acc[j][:, hc:]]
            dvs += [dv_acc[j][:, :hc], dv_acc[j][:, hc:]]
            pos += [j * hc, (2 * W - 1 - j) * hc]
        qp = (r * hc, (2 * W - 1 - r) * hc)
        ol, lsel = ltr.attn_fwd(ql, ks, vs, pos, qp, hc, True)
        if path == "bench":
            dql = torch.empty(ql.shape, dtype=torch.bfloat16, device="cuda")
            ltr.attn_bwd_accumulate(ql, dol, lsel, delta_ws, ks, vs, pos, dql, dks, dvs, qp, hc, True, do_dkdv=False, o=ol)
            ltr.attn_bwd_accumulate(ql, dol, lsel, delta_ws, ks, vs, pos, dql, dks, dvs, qp, hc, True, do_dq=False)
        else:
            delta = ltr.attn_delta(ol, dol)
            dql = torch.zeros(ql.shape, dtype=torch.float32, device="cuda")
            ltr.attn_bwd_accumulate(ql, dol, lsel, delta, ks, vs, pos, dql, dks, dvs, qp, hc, True)
        o[:, idx], dq[:, idx], lse[:, :, idx] = ol, dql.float(), lsel
    dk = torch.empty(kd.shape, dtype=torch.float32, device="cuda")
    dv = torch.empty(vd.shape, dtype=torch.float32, device="cuda")
    for r in range(W):
        dk[:, rp[r].cuda()], dv[:, rp[r].cuda()] = dk_acc[r], dv_acc[r]
    pos = torch.arange(S)
    oc, lsec, dqc, dkc, dvc = o.cpu(), lse.cpu(), dq.cpu(), dk.cpu(), dv.cpu()
    # edges: every half-chunk boundary (first / last key of each half-chunk; for rows, the segment split of the rank that
    # owns them), and a key inside the last 64-key tile that the diagonal of the last half-chunk sees
    half = [i * hc for i in range(1, 2 * W)]
    _check_rows(q, k, v, pos, pos, True, oc, lsec, do, dqc, n=30, edge_rows=[hc, S // 2, S - hc])
    _check_keys(q, k, v, oc, lsec, do, pos, pos, True, dkc, dvc, n=6, edge_keys=half + [S - 63])
    # softmax rows sum to one: sum_j dV_j == sum over the group's query heads and rows of dO
    lhs = dvc.double().sum(1)                                            # [B,Hkv,D]
    rhs = do.double().sum(1).reshape(B, Hkv, Hq // Hkv, D).sum(2)
    assert _rel(lhs, rhs) < 1e-2


def test_config3_full_ring_entry_point_fp32_kv_grads(ltr):
    """The same workload through the drop-in entry point: ring_attention_kernel with a LocalRing per rank (W = 8,
    zig-zag) and autograd, dK / dV summed over the 8 ranks in the ring's fp32 accumulators (RingKVGrads) and cast
    once."""
    g = torch.Generator().manual_seed(0)
    B, Hq, Hkv, D, S, W = 1, 32, 8, 128, 32768, 8
    mk = lambda h: torch.randn(B, S, h, D, generator=g).to(torch.bfloat16)
    q, k, v, do = mk(Hq), mk(Hkv), mk(Hkv), mk(Hq)
    rp = [orc.zigzag_positions(r, W, S) for r in range(W)]
    kv = [(k[:, p].cuda().requires_grad_(True), v[:, p].cuda().requires_grad_(True)) for p in rp]
    grads = ltr.RingKVGrads(kv)
    o = torch.empty(B, S, Hq, D, dtype=torch.bfloat16)
    lse = torch.empty(B, Hq, S)
    dq = torch.empty(B, S, Hq, D, dtype=torch.bfloat16)
    for r in range(W):
        ql = q[:, rp[r]].cuda().requires_grad_(True)
        ring = ltr.LocalRing(r, W, kv, causal=True, layout="zigzag", kv_grads=grads)
        ol = ltr.ring_attention_kernel(ql, kv[r][0], kv[r][1], ring, None)
        ol.backward(do[:, rp[r]].cuda())
        o[:, rp[r]], lse[:, :, rp[r]], dq[:, rp[r]] = ol.detach().cpu(), ring.last_lse.cpu(), ql.grad.cpu()
        assert kv[r][0].grad is None                      # nothing reaches k / v before finalize()
    grads.finalize()
    dk = torch.empty(B, S, Hkv, D, dtype=torch.bfloat16)
    dv = torch.empty(B, S, Hkv, D, dtype=torch.bfloat16)
    for r in range(W):
        dk[:, rp[r]], dv[:, rp[r]] = kv[r][0].grad.cpu(), kv[r][1].grad.cpu()
    pos = torch.arange(S)
    hc = S // (2 * W)
    _check_rows(q, k, v, pos, pos, True, o, lse, do, dq, n=20, seed=3, edge_rows=[hc, S // 2, S - hc])
    _check_keys(q, k, v, o, lse, do, pos, pos, True, dk, dv, n=6, seed=4, edge_keys=[i * hc for i in range(1, 2 * W, 3)] + [S - 63])
    rhs = do.double().sum(1).reshape(B, Hkv, Hq // Hkv, D).sum(2)
    assert _rel(dv.double().sum(1), rhs) < 1e-2


@pytest.mark.parametrize("path", ["accumulators", "bench", "fused_rope"])
def test_config4_full_rank15(ltr, path):
    """B=1, H=8, D=128, S=131072 as 16 chunks of 8192, bf16, causal, RoPE (base 10000) applied to
    q and k beforehand; rank 15's Q chunk against all 16 KV chunks: O, LSE, dQ and this rank's
    contribution to dK, dV of every chunk.  Paths "accumulators" and "bench" are those of test_config3_full_all_ranks;
    "fused_rope" hands the kernels the UN-rotated q chunk: the forward's prologue rotates it (positions 122880 ..
    131071; the rotated q must have the bits of the separate pass), the dQ kernel's epilogue rotates dQ back, and dQ is
    compared with the oracle's dQ of the rotated q carried through the conjugate rotation."""
    g = torch.Generator().manual_seed(0)
    B, H, D, S, W = 1, 8, 128, 131072, 16
    sl = S // W
    mk = lambda: torch.randn(B, S, H, D, generator=g).to(torch.bfloat16)
    q, k, v = mk(), mk(), mk()
    do = torch.randn(B, sl, H, D, generator=g).to(torch.bfloat16)
    # the angle table comes from the oracle so that both sides rotate by bit-identical angles: in fp32
    # the phase t*theta_i near t = 131071 moves by ~1e-2 rad per ulp of theta_i, and the CPU and GPU
    # pow() differ by an ulp (checked below with that bound; the reference has the same spread)
    fc_cpu = orc.precompute_freqs_cis(D, S)
    fc = fc_cpu.cuda()
    fc_gpu = ltr.precompute_freqs_cis(D, S, device="cuda").cpu()
    assert torch.equal(ltr.precompute_freqs_cis(D, S), fc_cpu) or (ltr.precompute_freqs_cis(D, S) - fc_cpu).abs().max() < 1e-6
    assert (torch.angle(fc_gpu * fc_cpu.conj())).abs().max() < 3e-2
    q_raw = q
    qd, kd = ltr.apply_rotary_emb(q.cuda(), k.cuda(), fc)
    vd = v.cuda()
    q, k = qd.cpu(), kd.cpu()                                              # the oracle sees the rotated bf16 inputs
    # RoPE itself against the oracle's restatement on a slice (positions near the top end)
    # (fp32 in and out: the bf16 cast would hide or amplify differences by one bf16 ulp)
    x = torch.randn(1, 64, 2, D, generator=g)
    ro_q, _ = orc.apply_rotary_emb(x, x, fc_cpu[S - 64:])
    rg_q, _ = ltr.apply_rotary_emb(x.cuda(), x.cuda(), fc[S - 64:])
    assert (rg_q.cpu() - ro_q).abs().max() < 1e-5, (rg_q.cpu() - ro_q).abs().max()
    q_unrot = q_raw[:, 15 * sl:].cuda() if path == "fused_rope" else None
    ql, dol = qd[:, 15 * sl:].contiguous(), do.cuda()
    ks = [kd[:, j * sl:(j + 1) * sl] for j in orc.ring_order(15, W)]
    vs = [vd[:, j * sl:(j + 1) * sl] for j in orc.ring_order(15, W)]
    pos0 = [j * sl for j in orc.ring_order(15, W)]
    if path == "fused_rope":
        table = ltr.rope_table(fc)
        q_rot = torch.empty_like(ql)
        ol, lsel = ltr.attn_fwd(q_unrot, ks, vs, pos0, 15 * sl, None, True, q_rope=table, q_rot_out=q_rot)
        assert torch.equal(q_rot, ql)
    else:
        ol, lsel = ltr.attn_fwd(ql, ks, vs, pos0, 15 * sl, None, True)
    dk = torch.zeros(kd.shape, dtype=torch.float32, device="cuda")
    dv = torch.zeros(vd.shape, dtype=torch.float32, device="cuda")
    dks = [dk[:, j * sl:(j + 1) * sl] for j in orc.ring_order(15, W)]
    dvs = [dv[:, j * sl:(j + 1) * sl] for j in orc.ring_order(15, W)]
    if path in ("bench", "fused_rope"):
        dq = torch.empty(ql.shape, dtype=torch.bfloat16, device="cuda")
        delta_ws = torch.empty(B, H, sl, dtype=torch.float32, device="cuda")
        ltr.attn_bwd_accumulate(ql, dol, lsel, delta_ws, ks, vs, pos0, dq, dks, dvs, 15 * sl, None, True, do_dkdv=False, o=ol,
                                dq_rope=table if path == "fused_rope" else None)
        ltr.attn_bwd_accumulate(ql, dol, lsel, delta_ws, ks, vs, pos0, dq, dks, dvs, 15 * sl, None, True, do_dq=False)
        if path == "fused_rope":
            # dq is the gradient of the un-rotated q; rotating it forward again gives the gradient of the rotated q (the
            # rotation is orthogonal), which is what the sampled-row check below computes
            dq = ltr.rope_one(dq, fc[15 * sl:])
    else:
        delta = ltr.attn_delta(ol, dol)
        dq = torch.zeros(ql.shape, dtype=torch.float32, device="cuda")
        ltr.attn_bwd_accumulate(ql, dol, lsel, delta, ks, vs, pos0, dq, dks, dvs, 15 * sl, None, True)
    qpos, kpos = torch.arange(sl) + 15 * sl, torch.arange(S)
    qc = q[:, 15 * sl:]
    oc, lsec = ol.cpu(), lsel.cpu()
    # edges: chunk boundaries of the ring (first / last key of a chunk), the first key of the diagonal chunk and a key in
    # the last tile the diagonal sees
    _check_rows(qc, k, v, qpos, kpos, True, oc, lsec, do, dq.cpu(), n=20, edge_rows=[sl // 2])
    _check_keys(qc, k, v, oc, lsec, do, qpos, kpos, True, dk.cpu(), dv.cpu(), n=6, edge_keys=[sl, 8 * sl, 15 * sl, S - 63])


def test_config5_full_ulysses_layout(ltr):
    """B=8, H=16, D=64, S=4096, bf16, non-causal; input sequence-sharded [B, S/4, H, D] over 4 ranks,
    permuted to head-sharded [B, S, H/4, D] (the all-to-all's stand-in), attention fwd+bwd on rank
    1's 4 heads, gradients permuted back to sequence shards; U(-1,1), seed 7."""
    g = torch.Generator().manual_seed(7)
    W, B, S, H, D = 4, 8, 4096, 16, 64
    mk = lambda: (torch.rand(W, B, S // W, H, D, generator=g) * 2 - 1).to(torch.bfloat16)
    q, k, v, do = mk(), mk(), mk(), mk()
    grp = ltr.LocalCPGroup(W)
    qd, kd, vd = (x.cuda().requires_grad_(True) for x in (q, k, v))
    qh, kh, vh = (ltr._all_to_all(x, 2, 1, grp) for x in (qd, kd, vd))        # [W, B, S, H/W, D]
    ref_q = orc.seq_all_to_all([q[r] for r in range(W)], 2, 1)
    assert torch.equal(qh[1].detach().cpu(), ref_q[1])
    r = 1
    o, lse = ltr.block_attention(qh[r], [kh[r]], [vh[r]], [0], 0, None, False)
    # head-sharded dO of rank r, then backward through attention and the exchange
    doh = ltr._all_to_all(do.cuda(), 2, 1, grp)[r]
    o.backward(doh)
    qf, kf, vf, dof = (orc.seq_all_to_all([x[j] for j in range(W)], 2, 1)[r] for x in (q, k, v, do))
    pos = torch.arange(S)
    oc, lsec = o.detach().cpu(), lse.cpu()
    # gradients arrive on the sequence shards: rank j's rows of head group r; permute back for the check
    dq_h = torch.cat([qd.grad[j][:, :, r * (H // W):(r + 1) * (H // W)] for j in range(W)], 1).cpu()
    dk_h = torch.cat([kd.grad[j][:, :, r * (H // W):(r + 1) * (H // W)] for j in range(W)], 1).cpu()
    dv_h = torch.cat([vd.grad[j][:, :, r * (H // W):(r + 1) * (H // W)] for j in range(W)], 1).cpu()
    _check_rows(qf, kf, vf, pos, pos, False, oc, lsec, dof, dq_h, n=24)
    _check_keys(qf, kf, vf, oc, lsec, dof, pos, pos, False, dk_h, dv_h, n=6)
    # heads outside group r received no gradient
    assert qd.grad[0][:, :, :r * (H // W)].abs().max() == 0


@pytest.mark.parametrize("keys,rows", [(256, 512), (128, 256)])
def test_head_dim_64_ring_share_both_block_sizes(ltr, keys, rows):
    """Head dim 64 at a size where the 256-key dK/dV blocks and 512-row dQ blocks are what the library runs: one zig-zag rank
    share (rank 2 of 4: half-chunks 2 and 5 of 8 x 2048 positions) of a causal GQA 8/2 sequence of 16384, B = 2, against all
    8 KV half-chunks in ring order, fp32 dK / dV accumulators, bf16 dQ with DELTA from O.  Both block sizes of all three
    kernels forced through the hint flags (the forward with the dQ kernel's rows per block); sampled rows (O, LSE, dQ) and sampled keys (dK, dV) against the oracle's closed form."""
    g = torch.Generator().manual_seed(5)
    B, Hq, Hkv, D, S, W = 2, 8, 2, 64, 16384, 4
    hc = S // (2 * W)
    q = torch.randn(B, S, Hq, D, generator=g).to(torch.bfloat16)
    k = torch.randn(B, S, Hkv, D, generator=g).to(torch.bfloat16)
    v = torch.randn(B, S, Hkv, D, generator=g).to(torch.bfloat16)
    r = 2
    qpos = orc.zigzag_positions(r, W, S)
    do = torch.randn(B, 2 * hc, Hq, D, generator=g).to(torch.bfloat16)
    kd, vd = k.cuda(), v.cuda()
    ql, dol = q[:, qpos].cuda(), do.cuda()
    order = []
    for j in orc.ring_order(r, W):
        order += [j, 2 * W - 1 - j]                      # the two half-chunks of rank j
    ks = [kd[:, i * hc:(i + 1) * hc] for i in order]
    vs = [vd[:, i * hc:(i + 1) * hc] for i in order]
    pos0 = [i * hc for i in order]
    qp = (r * hc, (2 * W - 1 - r) * hc)
    ol, lsel = ltr.attn_fwd(ql, ks, vs, pos0, qp, hc, True, fwd_rows=rows)     # the forward's block follows the dQ kernel's
    dk = torch.zeros(kd.shape, dtype=torch.float32, device="cuda")
    dv = torch.zeros(vd.shape, dtype=torch.float32, device="cuda")
    dks = [dk[:, i * hc:(i + 1) * hc] for i in order]
    dvs = [dv[:, i * hc:(i + 1) * hc] for i in order]
    dq = torch.empty(ql.shape, dtype=torch.bfloat16, device="cuda")
    delta_ws = torch.empty(B, Hq, 2 * hc, dtype=torch.float32, device="cuda")
    ltr.attn_bwd_accumulate(ql, dol, lsel, delta_ws, ks, vs, pos0, dq, dks, dvs, qp, hc, True, do_dkdv=False, o=ol, dq_rows=rows)
    ltr.attn_bwd_accumulate(ql, dol, lsel, delta_ws, ks, vs, pos0, dq, dks, dvs, qp, hc, True, do_dq=False, dkdv_keys=keys)
    kpos = torch.arange(S)
    oc, lsec = ol.cpu(), lsel.cpu()
    # edges: the segment split of the share's rows (q_split - 1 / q_split), 512-row tile edges, half-chunk boundaries of the keys
    _check_rows(q[:, qpos], k, v, qpos, kpos, True, oc, lsec, do, dq.cpu(), n=20, edge_rows=[hc, 512])
    _check_keys(q[:, qpos], k, v, oc, lsec, do, qpos, kpos, True, dk.cpu(), dv.cpu(), n=8, edge_keys=[256, 3 * hc, 6 * hc, 6 * hc - 63])


@pytest.mark.parametrize("Sq", [2048, 1900])
def test_head_dim_64_paired_512_row_blocks(ltr, Sq):
    """Head dim 64, one causal chunk, enough (batch, head) pairs that the 512-row blocks of the forward and dQ kernels are
    handed out in pairs (late q tile + early counterpart: 4 tiles -> 2 slots x 128 pairs = 256 blocks, one per CU), with a
    ragged last tile in the second case.  512 rows forced through the hint flags (the library's own choice at 2048); sampled
    rows and keys against the oracle's closed form."""
    g = torch.Generator().manual_seed(11 + Sq)
    B, Hq, Hkv, D = 4, 32, 8, 64
    q = torch.randn(B, Sq, Hq, D, generator=g).to(torch.bfloat16)
    k = torch.randn(B, Sq, Hkv, D, generator=g).to(torch.bfloat16)
    v = torch.randn(B, Sq, Hkv, D, generator=g).to(torch.bfloat16)
    do = torch.randn(B, Sq, Hq, D, generator=g).to(torch.bfloat16)
    qd, kd, vd, dod = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    o, lse = ltr.attn_fwd(qd, [kd], [vd], [0], 0, None, True, fwd_rows=512)
    o256, lse256 = ltr.attn_fwd(qd, [kd], [vd], [0], 0, None, True, fwd_rows=256)
    assert (o.float() - o256.float()).abs().max() <= 2e-2 and (lse - lse256).abs().max() <= 1e-3
    dq = torch.empty(qd.shape, dtype=torch.bfloat16, device="cuda")
    dk = torch.empty(kd.shape, dtype=torch.bfloat16, device="cuda")
    dv = torch.empty(vd.shape, dtype=torch.bfloat16, device="cuda")
    delta_ws = torch.empty(B, Hq, Sq, dtype=torch.float32, device="cuda")
    ltr.attn_bwd_accumulate(qd, dod, lse, delta_ws, [kd], [vd], [0], dq, [dk], [dv], 0, None, True, do_dkdv=False, o=o, dq_rows=512)
    ltr.attn_bwd_accumulate(qd, dod, lse, delta_ws, [kd], [vd], [0], dq, [dk], [dv], 0, None, True, do_dq=False)
    pos = torch.arange(Sq)
    oc, lsec = o.cpu(), lse.cpu()
    _check_rows(q, k, v, pos, pos, True, oc, lsec, do, dq.cpu(), n=30, edge_rows=[512, Sq - Sq % 512 or Sq])
    _check_keys(q, k, v, oc, lsec, do, pos, pos, True, dk.float().cpu(), dv.float().cpu(), n=8, edge_keys=[256, Sq - 63])
