"""Benchmark of the ring-attention hot path on one MI355X.

Default workload (the one the headline metric is quoted on): B=1, Hq=32, Hkv=8, D=128,
S=32768, bf16, causal, zig-zag assignment over 8 ranks; one "step" runs every rank's share
(forward over the 16 half-chunk KV table, DELTA, recompute backward with dK/dV accumulated
in fp32 across shares, final casts) so a step is the whole sequence's forward+backward.
Inputs are synthetic N(0,1) (seed 0) and resident in HBM before the timed region.

Prints ONE JSON line.  `value` is causal-adjusted TFLOP/s: 14*B*Hq*D*N_pairs flops (2 GEMMs
forward, 5 backward, unmasked pairs only) divided by the step time.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16 matrix peak
KERNEL_SOURCE = os.path.join(ROOT, "lightron_amd", "csrc", "ltr_attn.hip")
COUNTER_PROFILE = os.path.join(ROOT, "profiles", "bench_c3_counters.md")


def _measured_traffic(kernel):
    """HBM-side bytes per launch of `kernel` on config 3 as the rocprofv3 FETCH_SIZE / WRITE_SIZE runs recorded in
    profiles/bench_c3_counters.md measured them.  The profile names the sha256 of the kernel source it was taken from;
    when the source has changed since, the figure is stale and None is reported instead."""
    import hashlib
    import re
    try:
        text = open(COUNTER_PROFILE).read()
        digest = hashlib.sha256(open(KERNEL_SOURCE, "rb").read()).hexdigest()
    except OSError:
        return None, "no counter profile"
    m = re.search(r"^kernel-source-sha256: ([0-9a-f]{64})$", text, flags=re.M)
    t = re.search(r"^traffic-bytes-per-launch %s: ([0-9.e+]+)$" % re.escape(kernel), text, flags=re.M)
    if not m or not t:
        return None, "profiles/bench_c3_counters.md has no machine-readable traffic line for %s" % kernel
    if m.group(1) != digest:
        return None, "profiles/bench_c3_counters.md was taken from an older kernel source (stale)"
    return float(t.group(1)), "profiles/bench_c3_counters.md (rocprofv3 FETCH_SIZE/WRITE_SIZE, source sha256 %s)" % digest[:12]


def _workload(name):
    # (B, Hq, Hkv, D, S_total, W ranks, layout, causal, ranks to run, bwd)
    if name == "c3":
        return dict(B=1, Hq=32, Hkv=8, D=128, S=32768, W=8, layout="zigzag", causal=True,
                    ranks=list(range(8)), bwd=True,
                    desc="config 3: GQA 32/8 D=128 S=32768 bf16 causal, 8 zig-zag rank shares, fwd+bwd")
    if name == "c2":
        return dict(B=4, Hq=32, Hkv=32, D=128, S=8192, W=8, layout="contiguous", causal=True,
                    ranks=[7], bwd=False,
                    desc="config 2: B=4 H=32 D=128, last rank's Q chunk 1024 vs 8x1024 KV, bf16 causal, fwd")
    if name == "c4":
        return dict(B=1, Hq=8, Hkv=8, D=128, S=131072, W=16, layout="contiguous", causal=True,
                    ranks=[15], bwd=True,
                    desc="config 4: H=8 D=128 S=131072, rank 15's 8192-token Q chunk vs 16x8192 KV, fwd+bwd")
    if name == "c5":
        return dict(B=8, Hq=4, Hkv=4, D=64, S=4096, W=1, layout="contiguous", causal=False,
                    ranks=[0], bwd=True,
                    desc="config 5: B=8, 4 local heads of 16, D=64, S=4096, non-causal, fwd+bwd")
    if name == "s2k":
        return dict(B=8, Hq=32, Hkv=32, D=128, S=2048, W=1, layout="contiguous", causal=True,
                    ranks=[0], bwd=True,
                    desc="single-chunk causal attention (the Attention.forward / Ulysses local shape): B=8 H=32 D=128 S=2048, fwd+bwd")
    raise SystemExit("unknown workload %r" % name)


def _rank_positions(cfg, r):
    import torch
    W, S = cfg["W"], cfg["S"]
    if cfg["layout"] == "zigzag":
        hc = S // (2 * W)
        return torch.cat([torch.arange(r * hc, (r + 1) * hc), torch.arange((2 * W - 1 - r) * hc, (2 * W - r) * hc)])
    sl = S // W
    return torch.arange(r * sl, (r + 1) * sl)


def _n_pairs(cfg, r):
    import torch
    qp = _rank_positions(cfg, r)
    if not cfg["causal"]:
        return qp.numel() * cfg["S"]
    return int((qp + 1).sum())          # keys 0..pos visible


def _cpu_baseline(cfg, threads):
    """The oracle (the reference composition restated in torch) timed on the host cores on a
    bounded sample: one off-diagonal and one diagonal 2048x2048 block-step of the workload's
    head configuration, forward by the online-softmax recurrence and backward by autograd
    through it, fp32."""
    import torch
    from oracle import ring_attention_oracle as orc
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(0)
    blk = min(2048, cfg["S"])
    B, Hq, Hkv, D = cfg["B"], cfg["Hq"], cfg["Hkv"], cfg["D"]
    q = torch.randn(B, blk, Hq, D, generator=g).requires_grad_(True)
    k = torch.randn(B, blk, Hkv, D, generator=g).requires_grad_(True)
    v = torch.randn(B, blk, Hkv, D, generator=g).requires_grad_(True)
    do = torch.randn(B, blk, Hq, D, generator=g)
    pos = torch.arange(blk)
    flops = 0.0
    t_total = 0.0
    reps = 0
    cases = [(pos + blk, False), (pos, True)] if cfg["causal"] else [(pos, False)]
    t_start = time.time()
    while t_total < 10.0 and time.time() - t_start < 40.0:
        for qpos, diag in cases:
            t0 = time.time()
            o, _ = orc.ring_attention_recurrence(q, [(k, v)], qpos, [pos], cfg["causal"])
            if cfg["bwd"]:
                o.backward(do)
            t_total += time.time() - t0
            pairs = blk * (blk + 1) // 2 if diag else blk * blk
            flops += (14.0 if cfg["bwd"] else 4.0) * B * Hq * D * pairs
        reps += 1
    return {"value": flops / t_total / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": "%d x (%s) %dx%d block-steps, B=%d Hq=%d Hkv=%d D=%d, fp32 torch CPU, %s; %.1f s" % (
                reps, "off-diagonal + diagonal" if cfg["causal"] else "full", blk, blk, B, Hq, Hkv, D,
                "fwd + autograd bwd" if cfg["bwd"] else "fwd", t_total)}


def _bench_rope(args):
    """RoPE pre-pass of config 4 (q chunk of rank 15 and all of k, bf16, D=128): one launch of rope_kernel per
    tensor.  HBM bound: algorithmic bytes = read + write of every element plus one read of the (cos, sin) rows."""
    import torch
    import lightron_amd as la
    la._lib.load()
    dev = torch.device("cuda:0")
    B, H, D, S, Sq = 1, 8, 128, 131072, 8192
    g = torch.Generator().manual_seed(0)
    q = torch.randn(B, Sq, H, D, generator=g).to(torch.bfloat16).to(dev)
    k = torch.randn(B, S, H, D, generator=g).to(torch.bfloat16).to(dev)
    fc = la.precompute_freqs_cis(D, S, device=dev)
    fq = fc[S - Sq:]
    tq, tk = torch.view_as_real(fq).contiguous(), torch.view_as_real(fc).contiguous()
    from lightron_amd.layers import _rope_launch
    def step():
        _rope_launch(q, tq, False)
        _rope_launch(k, tk, False)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    evs = []
    t0 = time.perf_counter()
    for _ in range(args.steps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        _rope_launch(k, tk, False)
        e1.record()
        evs.append((e0, e1))
        _rope_launch(q, tq, False)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    k_ms = sum(a.elapsed_time(b) for a, b in evs) / len(evs)
    k_bytes = k.numel() * 4 + tk.numel() * 4          # bf16 in + bf16 out, fp32 table rows once
    tot_bytes = k_bytes + q.numel() * 4 + tq.numel() * 4
    out = {"metric": "RoPE pre-pass GB/s (config 4 shapes, bf16)", "value": round(tot_bytes / dt / 1e9, 1), "unit": "GB/s",
           "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(dt * 1e3, 4),
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "config 4 RoPE: q [1,8192,8,128] at positions 122880.., k [1,131072,8,128], bf16"},
           "roofline": {"bound": "hbm", "kernel": "rope_kernel<bf16>", "achieved": round(k_bytes / (k_ms * 1e-3) / 1e9, 1),
                        "peak": 8000.0, "unit": "GB/s", "frac": round(k_bytes / (k_ms * 1e-3) / 1e9 / 8000.0, 4), "traffic": None}}
    print(json.dumps(out), flush=True)


def _cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.lower().startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _device_report(la, torch, probe=True):
    """hipDeviceProp facts of the device plus what it sustains on the matrix pipe right now: a register-resident
    v_mfma_f32_32x32x16_bf16 loop on random and on constant operands, with the shader clock measured inside each."""
    import ctypes
    lib = la._lib.load()
    info = la._lib.DeviceInfo()
    la._lib.check(lib.ltr_device_info(ctypes.byref(info)), "ltr_device_info")
    rep = {"name": torch.cuda.get_device_properties(0).name, "arch": info.arch.decode(), "cus": info.compute_units,
           "clock_mhz": info.clock_khz // 1000, "memory_clock_mhz": info.memory_clock_khz // 1000,
           "memory_bus_bits": info.memory_bus_bits, "hbm_gib": round(info.hbm_bytes / 2**30, 1)}
    if not probe:
        return rep
    n = 8192 + (1 << 20)
    g = torch.Generator().manual_seed(1)
    ws = torch.empty(n, dtype=torch.uint8, device="cuda")
    ws[8192:] = ((torch.rand((n - 8192) // 2, generator=g) * 4 - 2).to(torch.bfloat16)).view(torch.uint8).cuda()
    iters = 200000
    stream = torch.cuda.current_stream().cuda_stream
    for key, rnd in (("random_operands", 1), ("constant_operands", 0)):
        best = None
        for _ in range(2):      # the first launch also ramps the clock
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            la._lib.check(lib.ltr_probe_mfma(ws.data_ptr(), n, iters, rnd, stream), "ltr_probe_mfma")
            e1.record()
            torch.cuda.synchronize()
            t = ws[:16].view(torch.int64).cpu()
            # rate: all waves' MFMAs over the launch's duration (HIP events); clock: shader ticks against the 100 MHz wall
            # clock over the loop of ONE wave (the two waves of a SIMD do not alternate: the older one runs its loop at the
            # pipe's full rate, then the other; both tick counts cover the same interval, so their ratio is the clock)
            ms = e0.elapsed_time(e1)
            cur = {"tflops": round(info.compute_units * 8 * iters * 4 * 32768.0 / (ms * 1e-3) / 1e12, 1),
                   "shader_clock_mhz": round(t[1].item() / (t[0].item() / 100e6) / 1e6, 0), "ms": round(ms, 3)}
            best = cur if best is None or cur["tflops"] > best["tflops"] else best
        rep["mfma_loop_" + key] = best
    return rep


def _run_attention(la, torch, cfg, steps, warmup, data="randn", min_warm_s=0.0, min_timed_s=0.0):
    """Times `steps` steps of one workload after `warmup` untimed ones; inputs are resident in HBM before the timed
    region.  Returns the step time, the credited flops and the average launch time of each kernel (HIP events on the
    stream the kernels are launched on).  data="zeros" replaces the workload's N(0,1) inputs by zeros (same kernels, same
    instruction stream, no toggling operand bits): only used by _data_dependence.
    min_warm_s / min_timed_s: workloads whose step takes well under a millisecond are over before the device, idle while
    the host generated the inputs, has settled (measured: config 2 849 TFLOP/s with 2 + 5 steps, 1066 after 100 ms of
    work); the untimed steps then go on until min_warm_s have passed, and the timed region covers at least min_timed_s
    (the numbers of steps actually run are returned)."""
    dev = torch.device("cuda:0")
    B, Hq, Hkv, D, S, W = (cfg[x] for x in ("B", "Hq", "Hkv", "D", "S", "W"))
    causal, bwd = cfg["causal"], cfg["bwd"]
    sl = S // W

    # synthetic inputs, generated on the CPU in the order q, k, v, dO, stored rank-major [W, B, S_l, H, D]
    g = torch.Generator().manual_seed(0)
    def mk(h):
        full = torch.randn(B, S, h, D, generator=g).to(torch.bfloat16)
        if data == "zeros":
            full.zero_()
        return torch.stack([full[:, _rank_positions(cfg, r)] for r in range(W)], 0).to(dev)
    q_all, k_all, v_all = mk(Hq), mk(Hkv), mk(Hkv)
    do_all = mk(Hq) if bwd else None

    # per-rank chunk tables in the reference's visiting order
    tables = {}
    for r in cfg["ranks"]:
        ks, vs, pos = [], [], []
        for j in [(r - s) % W for s in range(W)]:
            if cfg["layout"] == "zigzag":
                hc = sl // 2
                for half, p0 in ((slice(0, hc), j * hc), (slice(hc, sl), (2 * W - 1 - j) * hc)):
                    ks.append(k_all[j][:, half]); vs.append(v_all[j][:, half]); pos.append(p0)
            else:
                ks.append(k_all[j]); vs.append(v_all[j]); pos.append(j * sl)
        if cfg["layout"] == "zigzag":
            qp, qsplit = (r * (sl // 2), (2 * W - 1 - r) * (sl // 2)), sl // 2
        else:
            qp, qsplit = (r * sl, r * sl), sl
        tables[r] = (ks, vs, pos, qp, qsplit)

    o_all = torch.empty_like(q_all)
    lse_all = torch.empty(W, B, Hq, sl, dtype=torch.float32, device=dev)
    if bwd:
        # every rank's call holds all KV chunks its queries see, so the dQ kernel writes bf16 dQ itself (LTR_DQ_BF16)
        dq_out = torch.empty(q_all.shape, dtype=torch.bfloat16, device=dev)
        delta_ws = torch.empty(B, Hq, sl, dtype=torch.float32, device=dev)
        # dK / dV: fp32 accumulators summed over the rank shares and cast at the end; when the workload is ONE share that
        # holds the whole sequence (config 5) the kernel writes the bf16 results itself (LTR_DKDV_BF16)
        dkdv_direct = W == 1 and len(cfg["ranks"]) == 1
        acc_dtype = torch.bfloat16 if dkdv_direct else torch.float32
        dk_acc = torch.empty(k_all.shape, dtype=acc_dtype, device=dev)
        dv_acc = torch.empty(v_all.shape, dtype=acc_dtype, device=dev)

    def acc_views(r, acc):
        out = []
        for j in [(r - s) % W for s in range(W)]:
            if cfg["layout"] == "zigzag":
                hc = sl // 2
                out += [acc[j][:, :hc], acc[j][:, hc:]]
            else:
                out.append(acc[j])
        return out

    ev = {"fwd": [], "dkdv": [], "dq": []}

    def timed_call(key, timed, fn):
        if not timed:
            return fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        r = fn()
        e1.record()
        ev[key].append((e0, e1))
        return r

    def step(timed):
        if bwd and not dkdv_direct:
            dk_acc.zero_(); dv_acc.zero_()
        for r in cfg["ranks"]:
            ks, vs, pos, qp, qsplit = tables[r]
            timed_call("fwd", timed, lambda: la.attn_fwd(q_all[r], ks, vs, pos, qp, qsplit, causal, out=o_all[r],
                                                         lse=lse_all[r]))
            if bwd:
                dks, dvs = acc_views(r, dk_acc), acc_views(r, dv_acc)
                # the two backward kernels are enqueued by two calls so each can be timed on its own; the dQ kernel
                # goes first and also produces DELTA = rowsum(dO * O) for the dK/dV kernel (LTR_DELTA_FROM_O)
                timed_call("dq", timed, lambda: la.attn_bwd_accumulate(
                    q_all[r], do_all[r], lse_all[r], delta_ws, ks, vs, pos, dq_out[r], dks, dvs, qp, qsplit, causal,
                    do_dkdv=False, o=o_all[r]))
                timed_call("dkdv", timed, lambda: la.attn_bwd_accumulate(
                    q_all[r], do_all[r], lse_all[r], delta_ws, ks, vs, pos, dq_out[r], dks, dvs, qp, qsplit, causal,
                    do_dq=False))
        if bwd and not dkdv_direct:
            la.cast_to_bf16(dk_acc); la.cast_to_bf16(dv_acc)

    n_warm, t_w = 0, time.perf_counter()
    while n_warm < warmup or time.perf_counter() - t_w < min_warm_s:
        step(False)
        n_warm += 1
        if n_warm >= warmup:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    if min_timed_s > 0:
        t1 = time.perf_counter()           # one more untimed step sizes the timed region
        step(False)
        torch.cuda.synchronize()
        n_warm += 1
        steps = max(steps, int(math.ceil(min_timed_s / max(time.perf_counter() - t1, 1e-6))))
    t0 = time.perf_counter()
    for _ in range(steps):
        step(True)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps

    pairs = sum(_n_pairs(cfg, r) for r in cfg["ranks"])
    f_fwd = 4.0 * B * Hq * D * pairs
    f_total = f_fwd * (3.5 if bwd else 1.0)
    avg = lambda key: sum(a.elapsed_time(b) for a, b in ev[key]) / len(ev[key])
    fwd_ms = avg("fwd")
    launches = len(cfg["ranks"])
    f_share = f_fwd / launches                      # forward flops of one launch (one rank's share)
    kernels = {"fwd_bf16_kernel": {"ms_per_launch": round(fwd_ms, 4), "algorithmic_tflops": round(f_share / fwd_ms / 1e9, 2),
                                   "gemms_credited": 2, "gemms_executed": 2}}
    if bwd:
        # credited backward work is 5 GEMMs (S, dP, dV, dK, dQ); the dQ kernel recomputes S and dP
        dkdv_ms, dq_ms = avg("dkdv"), avg("dq")
        kernels["bwd_dkdv_kernel"] = {"ms_per_launch": round(dkdv_ms, 4), "gemms_credited": 4, "gemms_executed": 4,
                                      "algorithmic_tflops": round(2.0 * f_share / dkdv_ms / 1e9, 2)}
        kernels["bwd_dq_kernel"] = {"ms_per_launch": round(dq_ms, 4), "gemms_credited": 1, "gemms_executed": 3,
                                    "algorithmic_tflops": round(0.5 * f_share / dq_ms / 1e9, 2),
                                    "executed_tflops": round(1.5 * f_share / dq_ms / 1e9, 2)}
        # template arguments: head dim, 32-key halves per wave (2 = the 256-key blocks the library picks for long head-dim-64 streams)
        dom, dom_ms, dom_flops = "bwd_dkdv_kernel<%d, %d>" % (D, 2 if (D == 64 and not causal and S >= 4096) else 1), dkdv_ms, 2.0 * f_share
    else:
        dom, dom_ms, dom_flops = "fwd_bf16_kernel<%d, 1>" % D, fwd_ms, f_share
    return {"dt": dt, "f_total": f_total, "kernels": kernels, "launches": launches, "steps": steps, "warmup": n_warm,
            "dominant": (dom, dom_flops / (dom_ms * 1e-3) / 1e12)}


def _data_dependence(la, torch, cfg):
    """The same three kernels on one rank share of the workload, once on its N(0,1) inputs and once on all-zero inputs
    (identical launches and instruction streams).  Executed TFLOP/s of each kernel: on zeros the chip keeps its full
    clock, on random data the matrix pipe's switching activity runs it into the power limit - the gap between the
    two is the clock, not the kernels' schedule."""
    share = dict(cfg, ranks=cfg["ranks"][:1])
    out = {"what": "executed TFLOP/s per kernel, one rank share, same launches on N(0,1) inputs and on all-zero inputs"}
    for data in ("randn", "zeros", "randn", "zeros"):
        r = _run_attention(la, torch, share, 6, 3, data=data, min_warm_s=0.3, min_timed_s=0.1)
        k = r["kernels"]
        cur = {"fwd_bf16_kernel": k["fwd_bf16_kernel"]["algorithmic_tflops"]}
        if cfg["bwd"]:
            cur["bwd_dkdv_kernel"] = k["bwd_dkdv_kernel"]["algorithmic_tflops"]
            cur["bwd_dq_kernel"] = k["bwd_dq_kernel"]["executed_tflops"]
        key = "n01_inputs" if data == "randn" else "zero_inputs"
        out[key] = {n: max(v, out.get(key, {}).get(n, 0.0)) for n, v in cur.items()}
    return out


def _run_c4_rope(la, torch, steps, warmup):
    """Config 4's RoPE on the q side, timed both ways on the launches it touches (K is rotated beforehand in both):
    separate passes (ltr_rope_apply on q, forward, dQ kernel, conjugate ltr_rope_apply on dQ) against the fused prologue /
    epilogue (forward with LTR_ROPE_Q, dQ kernel with LTR_ROPE_DQ).  Also times the one-off K pass."""
    from lightron_amd.layers import _rope_launch
    dev = torch.device("cuda:0")
    B, H, D, S, W = 1, 8, 128, 131072, 16
    sl = S // W
    g = torch.Generator().manual_seed(0)
    q = torch.randn(B, sl, H, D, generator=g).to(torch.bfloat16).to(dev)
    k = torch.randn(B, S, H, D, generator=g).to(torch.bfloat16).to(dev)
    v = torch.randn(B, S, H, D, generator=g).to(torch.bfloat16).to(dev)
    do = torch.randn(B, sl, H, D, generator=g).to(torch.bfloat16).to(dev)
    table = la.rope_table(la.precompute_freqs_cis(D, S, device=dev))
    tq = table[15 * sl:].contiguous()
    order = [(15 - s) % W for s in range(W)]
    k_rot = _rope_launch(k, table, False)
    ks = [k_rot[:, j * sl:(j + 1) * sl] for j in order]
    vs = [v[:, j * sl:(j + 1) * sl] for j in order]
    pos = [j * sl for j in order]
    o = torch.empty_like(q)
    lse = torch.empty(B, H, sl, dtype=torch.float32, device=dev)
    delta = torch.empty_like(lse)
    dq = torch.empty_like(q)
    q_rot = torch.empty_like(q)
    dk = [torch.empty(0)] * W   # the dK/dV kernel is not part of this comparison

    def separate():
        qr = _rope_launch(q, tq, False)
        la.attn_fwd(qr, ks, vs, pos, 15 * sl, None, True, out=o, lse=lse)
        la.attn_bwd_accumulate(qr, do, lse, delta, ks, vs, pos, dq, ks, vs, 15 * sl, None, True, do_dkdv=False, o=o)
        return _rope_launch(dq, tq, True)

    def fused():
        la.attn_fwd(q, ks, vs, pos, 15 * sl, None, True, out=o, lse=lse, q_rope=table, q_rot_out=q_rot)
        la.attn_bwd_accumulate(q_rot, do, lse, delta, ks, vs, pos, dq, ks, vs, 15 * sl, None, True, do_dkdv=False, o=o,
                               dq_rope=table)
        return dq

    def timed(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps

    t_sep, t_fus = timed(separate), timed(fused)
    t_sep2, t_fus2 = timed(separate), timed(fused)
    t_k = timed(lambda: _rope_launch(k, table, False))
    return {"what": "config 4, q side: rope(q) + forward + dQ kernel + conj rope(dQ) as separate passes against the fused "
                    "prologue / epilogue; K is rotated once beforehand in both",
            "separate_ms": round(min(t_sep, t_sep2), 4), "fused_ms": round(min(t_fus, t_fus2), 4),
            "k_pass_ms": round(t_k, 4)}


def _bench_mfma_ceiling(args):
    """What the device sustains on the matrix pipe, for the record beside the attention numbers: the register-resident
    MFMA loop of ltr_probe_mfma on random and constant operands with the shader clock of each, and the vendor library's
    bf16 GEMM (torch.matmul, 8192^3) on N(0,1) inputs."""
    import torch
    import lightron_amd as la
    torch.cuda.set_device(0)
    rep = _device_report(la, torch)
    a = torch.randn(8192, 8192, device="cuda", dtype=torch.bfloat16)
    b = torch.randn(8192, 8192, device="cuda", dtype=torch.bfloat16)
    for _ in range(5):
        a @ b
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        a @ b
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / args.steps
    rep["library_gemm_bf16_8192"] = {"tflops": round(2 * 8192.0**3 / ms / 1e9, 1), "ms": round(ms, 4)}
    best = rep["mfma_loop_random_operands"]["tflops"]
    out = {"metric": "sustained bf16 MFMA rate of the device (register-resident v_mfma_f32_32x32x16_bf16 loop, random operands)",
           "value": best, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": None,
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
           "config": {"workload": "matrix-pipe ceiling probe: one block of 8 waves per CU, 4 MFMA chains per wave"},
           "frac_of_mfma_peak": round(best / MFMA_BF16_PEAK_TFLOPS, 4), "device": rep}
    print(json.dumps(out), flush=True)


def _bench_dq_atomics(args):
    """The rate at which 64 x 128 fp32 partial dQ tiles can be added into memory with global atomics (ltr_probe_atomic_tile_add):
    what a backward that produced dQ inside the key-owning blocks would need, beside what it needs at the dK/dV kernel's
    speed."""
    import torch
    import lightron_amd as la
    torch.cuda.set_device(0)
    lib = la._lib.load()
    n = 8192 + (1 << 20)
    g = torch.Generator().manual_seed(1)
    ws = torch.empty(n, dtype=torch.uint8, device="cuda")
    ws[8192:] = ((torch.rand((n - 8192) // 2, generator=g) * 4 - 2).to(torch.bfloat16)).view(torch.uint8).cuda()
    dst = torch.zeros(32, 4096, 128, dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    steps = 512
    res = {}
    for key, with_mfma in (("atomic_adds_only", 0), ("atomic_adds_between_40_mfma_per_wave", 1)):
        best = None
        for _ in range(3):
            dst.zero_()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            la._lib.check(lib.ltr_probe_atomic_tile_add(dst.data_ptr(), dst.numel(), ws.data_ptr(), n, steps, with_mfma, stream),
                          "ltr_probe_atomic_tile_add")
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
            best = ms if best is None or ms < best else best
        ok = bool((dst == steps / 8).all().item())
        res[key] = {"ms": round(best, 3), "us_per_tile_per_block": round(best * 1e3 / steps, 3),
                    "payload_TB_per_s": round(256 * steps * 32768 / (best * 1e-3) / 1e12, 3), "sums_correct": ok}
    # MFMA-only time of the same loop, for the share of the adds in the combined run: 40 MFMA per wave and step
    need = {"step_us_at_dkdv_speed": 2.06, "payload_TB_per_s_needed": round(256 * 32768 / 2.06e-6 / 1e12, 2),
            "note": "a 5-GEMM step of 64 rows x 128 keys x 4 slices per CU takes about 2.06 us at 1300 TFLOP/s; one 32 KiB tile add per step"}
    out = {"metric": "fp32 global-atomic tile-add rate (partial dQ of a fused backward)", "value": res["atomic_adds_only"]["payload_TB_per_s"],
           "unit": "TB/s", "n_gpus": 1, "steps": steps, "warmup": 0, "ms_per_step": None, "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "256 blocks x 8 waves, each block adds one 64 x 128 fp32 tile per step into a [32, 4096, 128] buffer shared like dQ"},
           "results": res, "needed_by_a_fused_backward": need}
    print(json.dumps(out), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c3", choices=["c2", "c3", "c4", "c5", "s2k", "rope", "mfma_ceiling", "dq_atomics"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-others", action="store_true", help="skip the short runs of the other workloads and the device probe")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        raise SystemExit("bench.py: this build runs on ONE GPU (no collectives, no sharding across GPUs); "
                         "run with --gpus 1")
    import torch
    import lightron_amd as la
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.workload == "rope":
        return _bench_rope(args)
    if args.workload == "mfma_ceiling":
        return _bench_mfma_ceiling(args)
    if args.workload == "dq_atomics":
        return _bench_dq_atomics(args)
    la._lib.load()
    torch.cuda.set_device(0)
    cfg = _workload(args.workload)
    # the headline workload: exactly --warmup untimed and --steps timed steps (35 ms each: the device has settled after
    # the warm-up); the sub-millisecond workloads warm up for at least 0.3 s ("warmup" reports the steps that took)
    res = _run_attention(la, torch, cfg, args.steps, args.warmup, min_warm_s=0.0 if args.workload == "c3" else 0.3)
    dt, f_total, bwd = res["dt"], res["f_total"], cfg["bwd"]
    tflops = f_total / dt / 1e12
    dom, achieved = res["dominant"]
    traffic, traffic_source = (None, None)
    if args.workload == "c3":
        traffic, traffic_source = _measured_traffic(dom)
    out = {
        "metric": ("ring-attn fwd+bwd causal TFLOP/s at S=32k bf16, 1 GPU; % of MFMA peak" if args.workload == "c3" else
                   "attention %s causal-adjusted TFLOP/s, 1 GPU; %% of MFMA peak" % ("fwd+bwd" if bwd else "fwd")),
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": res["warmup"],
        "ms_per_step": round(dt * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": cfg["desc"], "B": cfg["B"], "Hq": cfg["Hq"], "Hkv": cfg["Hkv"], "D": cfg["D"], "S": cfg["S"],
                   "ranks": res["launches"], "layout": cfg["layout"], "causal": cfg["causal"], "flops_per_step": f_total},
        "frac_of_mfma_peak": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4),
        "kernels": res["kernels"],
        "roofline": {"bound": "mfma", "kernel": dom, "achieved": round(achieved, 2), "peak": MFMA_BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4),
                     "traffic": traffic, "traffic_source": traffic_source},
    }
    if not args.no_others:
        # the other workloads, outside the timed region of the headline: a few steps each
        others = {}
        for name in ("c2", "c4", "c5", "s2k"):
            if name == args.workload:
                continue
            torch.cuda.empty_cache()
            ocfg = _workload(name)
            r = _run_attention(la, torch, ocfg, 5, 2, min_warm_s=0.3, min_timed_s=0.15)
            tf = r["f_total"] / r["dt"] / 1e12
            others[name] = {"workload": ocfg["desc"], "tflops": round(tf, 1), "ms_per_step": round(r["dt"] * 1e3, 3),
                            "steps": r["steps"], "warmup": r["warmup"],
                            "frac_of_mfma_peak": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
                            "kernel_ms": {k: v["ms_per_launch"] for k, v in r["kernels"].items()},
                            "dominant_kernel_frac": round(r["dominant"][1] / MFMA_BF16_PEAK_TFLOPS, 4)}
        torch.cuda.empty_cache()
        others["c4_rope"] = _run_c4_rope(la, torch, 5, 2)
        out["other_workloads"] = others
        torch.cuda.empty_cache()
        out["data_dependence"] = _data_dependence(la, torch, cfg)
    out["device"] = _device_report(la, torch, probe=not args.no_others)
    if "mfma_loop_random_operands" in out["device"]:
        # beside the fraction of the published peak: the fraction of what a pure MFMA loop sustains on THIS box on random data
        ceil = out["device"]["mfma_loop_random_operands"]["tflops"]
        out["frac_of_measured_mfma_ceiling"] = round(tflops / ceil, 4)
        out["roofline"]["frac_of_measured_mfma_ceiling"] = round(achieved / ceil, 4)
    if not args.no_cpu_baseline:
        # the host's cores as the box presents them; OMP_NUM_THREADS (set on the GPU boxes to the job's CPU share) caps
        # the threads actually used
        host_cores = os.cpu_count() or 1
        threads = int(os.environ["OMP_NUM_THREADS"]) if os.environ.get("OMP_NUM_THREADS", "").isdigit() else host_cores
        threads = max(1, min(threads, host_cores))
        base = _cpu_baseline(cfg, threads)
        base.update({"threads": threads, "host_cores": host_cores, "cpu_model": _cpu_model()})
        out["cpu_baseline"] = base
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
