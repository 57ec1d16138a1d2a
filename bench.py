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
    lib = la._lib.load_probe()      # the measurement library (include/ltr_probe.h), not the product
    info = la._lib.DeviceInfo()
    if lib.ltr_device_info(ctypes.byref(info)) != 0:
        raise RuntimeError("ltr_device_info failed")
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
            if lib.ltr_probe_mfma(ws.data_ptr(), n, iters, rnd, stream) != 0:
                raise RuntimeError("ltr_probe_mfma failed")
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

    # the kernels these launches run, as the library itself reports them (ltr_attn_plan: the function that sizes the launches)
    ks0, _, pos0_, qp0_, qsplit0_ = tables[cfg["ranks"][0]]
    plan = la.attn_plan(B, Hq, Hkv, D, sl, [k.shape[1] for k in ks0], pos0_, qp0_, qsplit0_, causal)

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
    kernels = {"fwd_bf16_kernel": {"name": plan["fwd"]["kernel"], "ms_per_launch": round(fwd_ms, 4),
                                   "algorithmic_tflops": round(f_share / fwd_ms / 1e9, 2), "gemms_credited": 2, "gemms_executed": 2}}
    if bwd:
        # credited backward work is 5 GEMMs (S, dP, dV, dK, dQ); the dQ kernel recomputes S and dP
        dkdv_ms, dq_ms = avg("dkdv"), avg("dq")
        kernels["bwd_dkdv_kernel"] = {"name": plan["dkdv"]["kernel"], "ms_per_launch": round(dkdv_ms, 4), "gemms_credited": 4,
                                      "gemms_executed": 4, "algorithmic_tflops": round(2.0 * f_share / dkdv_ms / 1e9, 2)}
        kernels["bwd_dq_kernel"] = {"name": plan["dq"]["kernel"], "ms_per_launch": round(dq_ms, 4), "gemms_credited": 1, "gemms_executed": 3,
                                    "algorithmic_tflops": round(0.5 * f_share / dq_ms / 1e9, 2),
                                    "executed_tflops": round(1.5 * f_share / dq_ms / 1e9, 2)}
        dom, dom_ms, dom_flops = plan["dkdv"]["kernel"], dkdv_ms, 2.0 * f_share
    else:
        dom, dom_ms, dom_flops = plan["fwd"]["kernel"], fwd_ms, f_share
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


def _run_ref_default(la, torch):
    """The reference's own default shapes (config/config_tinystories.json:21-23 with the gpt2 model: micro-batch 4, 12
    heads of 64, sequence 128; trainer.py:48-55 runs forward and autograd backward): one causal attention call through the
    drop-in (block_attention, autograd) beside the library attention the reference calls there
    (F.scaled_dot_product_attention, model/model.py:193), microseconds per forward+backward call with the host side
    included (wall clock over many calls, one synchronisation at the end), S = 128, 256, 512."""
    import torch.nn.functional as F
    dev = torch.device("cuda:0")
    B, H, D = 4, 12, 64
    out = {"what": "us per forward+backward call, host side included, bf16 causal B=4 H=12 D=64; best of 3 interleaved runs of 300 calls"}

    def wall(fn, n=300, warm=60):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e6

    for S in (128, 256, 512):
        g = torch.Generator().manual_seed(S)
        q, k, v = (torch.randn(B, S, H, D, generator=g).to(torch.bfloat16).to(dev).requires_grad_(True) for _ in range(3))
        do = torch.randn(B, S, H, D, generator=g).to(torch.bfloat16).to(dev)
        qt, kt, vt = (x.detach().transpose(1, 2).requires_grad_(True) for x in (q, k, v))     # [B, H, S, D] views for SDPA
        dot = do.transpose(1, 2)

        def ours():
            o, _ = la.block_attention(q, [k], [v], [0], causal=True)
            o.backward(do)
            q.grad = k.grad = v.grad = None

        def library():
            o = F.scaled_dot_product_attention(qt, kt, vt, is_causal=True)
            o.backward(dot)
            qt.grad = kt.grad = vt.grad = None

        def ours_fwd():
            with torch.no_grad():
                la.block_attention(q, [k], [v], [0], causal=True)

        def library_fwd():
            with torch.no_grad():
                F.scaled_dot_product_attention(qt, kt, vt, is_causal=True)

        t = {"block_attention_us": [], "library_sdpa_us": [], "block_attention_fwd_only_us": [], "library_sdpa_fwd_only_us": []}
        for _ in range(3):
            t["block_attention_us"].append(wall(ours))
            t["library_sdpa_us"].append(wall(library))
            t["block_attention_fwd_only_us"].append(wall(ours_fwd))
            t["library_sdpa_fwd_only_us"].append(wall(library_fwd))
        out["S%d" % S] = {key: round(min(vals), 1) for key, vals in t.items()}
    return out


def _run_c3_stepwise(la, torch, steps, warmup):
    """Config 3, one zig-zag rank share (rank 0), in the call pattern of a real ring, where KV chunks arrive one at a time:
    the forward is one launch per half-chunk with the (O, LSE) merge fused into the kernel's epilogue (LTR_MERGE, fp32 O
    and LSE read-modify-written by every launch after the first), the backward one ltr_attn_bwd per half-chunk adding
    into fp32 dQ / dK / dV accumulators (DELTA from one ltr_attn_bwd_delta launch), then the casts.  Beside it the same
    share through one launch per kernel over the 16-entry chunk table, which is what the headline times."""
    dev = torch.device("cuda:0")
    cfg = _workload("c3")
    B, Hq, Hkv, D, S, W = (cfg[x] for x in ("B", "Hq", "Hkv", "D", "S", "W"))
    sl, hc, r = S // W, S // (2 * W), 0
    g = torch.Generator().manual_seed(0)
    def mk(h, n):
        return torch.randn(B, n, h, D, generator=g).to(torch.bfloat16).to(dev)
    q, k, v, do = mk(Hq, sl), mk(Hkv, S), mk(Hkv, S), mk(Hq, sl)
    # the ring's visiting order (r, r-1, ... mod W), two half-chunks per rank; k / v here are stored in POSITION order
    order = [(r - s_) % W for s_ in range(W)]
    halves = [h_ for j in order for h_ in (j, 2 * W - 1 - j)]
    ks = [k[:, h_ * hc:(h_ + 1) * hc] for h_ in halves]
    vs = [v[:, h_ * hc:(h_ + 1) * hc] for h_ in halves]
    pos = [h_ * hc for h_ in halves]
    qp, qsplit = (r * hc, (2 * W - 1 - r) * hc), hc
    o32 = torch.empty(B, sl, Hq, D, dtype=torch.float32, device=dev)
    o16 = torch.empty(B, sl, Hq, D, dtype=torch.bfloat16, device=dev)
    lse = torch.empty(B, Hq, sl, dtype=torch.float32, device=dev)
    dq32 = torch.empty(B, sl, Hq, D, dtype=torch.float32, device=dev)
    dq16 = torch.empty(B, sl, Hq, D, dtype=torch.bfloat16, device=dev)
    dk32, dv32 = torch.empty(k.shape, dtype=torch.float32, device=dev), torch.empty(v.shape, dtype=torch.float32, device=dev)
    dks = [dk32[:, h_ * hc:(h_ + 1) * hc] for h_ in halves]
    dvs = [dv32[:, h_ * hc:(h_ + 1) * hc] for h_ in halves]
    delta = torch.empty(B, Hq, sl, dtype=torch.float32, device=dev)
    n = len(ks)

    def stepwise_fwd(g_=1):
        # g_ KV half-chunks per launch: 1 = one launch per half-chunk (16 steps), 2 = one per rank chunk (the 8 steps of this ring)
        la.attn_fwd(q, ks[:g_], vs[:g_], pos[:g_], qp, qsplit, True, out=o32, lse=lse)
        for i in range(g_, n, g_):
            la.attn_fwd(q, ks[i:i + g_], vs[i:i + g_], pos[i:i + g_], qp, qsplit, True, out=o32, lse=lse, merge=True)

    def stepwise_bwd(g_=1):
        dq32.zero_(); dk32.zero_(); dv32.zero_()
        d = la.attn_delta(o32, do)
        for i in range(0, n, g_):
            la.attn_bwd_accumulate(q, do, lse, d, ks[i:i + g_], vs[i:i + g_], pos[i:i + g_], dq32, dks[i:i + g_], dvs[i:i + g_], qp, qsplit, True)
        la.cast_to_bf16(dq32); la.cast_to_bf16(dk32); la.cast_to_bf16(dv32)

    def table_fwd():
        la.attn_fwd(q, ks, vs, pos, qp, qsplit, True, out=o16, lse=lse)

    def table_bwd():
        dk32.zero_(); dv32.zero_()
        la.attn_bwd_accumulate(q, do, lse, delta, ks, vs, pos, dq16, dks, dvs, qp, qsplit, True, o=o16)
        la.cast_to_bf16(dk32); la.cast_to_bf16(dv32)

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

    table_fwd()      # o16 / lse for the table backward
    res = {}
    for _ in range(2):
        for key, fn in (("table_fwd_ms", table_fwd), ("table_bwd_ms", table_bwd), ("stepwise_fwd_ms", stepwise_fwd),
                        ("stepwise_bwd_ms", stepwise_bwd), ("rank_chunk_steps_fwd_ms", lambda: stepwise_fwd(2)),
                        ("rank_chunk_steps_bwd_ms", lambda: stepwise_bwd(2))):
            ms = timed(fn)
            res[key] = min(ms, res.get(key, ms))
    pairs = _n_pairs(cfg, r)
    f_share = 14.0 * B * Hq * D * pairs
    t_step, t_tab = res["stepwise_fwd_ms"] + res["stepwise_bwd_ms"], res["table_fwd_ms"] + res["table_bwd_ms"]
    out = {"what": "config 3, rank 0's share: one launch per ring step (16 forward launches with LTR_MERGE into fp32 O/LSE, 16 "
                   "ltr_attn_bwd calls into fp32 dQ/dK/dV, zero-fills, DELTA pass and casts included) beside one launch per "
                   "kernel over the 16-entry chunk table",
           "launches_per_share": {"stepwise": 16 + 1 + 2 * 16 + 6, "rank_chunk_steps": 8 + 1 + 2 * 8 + 6, "table": 1 + 2 + 4}}
    out.update({key: round(val, 4) for key, val in res.items()})
    t_rank = res["rank_chunk_steps_fwd_ms"] + res["rank_chunk_steps_bwd_ms"]
    out.update({"stepwise_ms": round(t_step, 4), "table_ms": round(t_tab, 4), "stepwise_over_table": round(t_step / t_tab, 4),
                "stepwise_tflops": round(f_share / t_step / 1e9, 1), "table_tflops": round(f_share / t_tab / 1e9, 1),
                # the same with one launch per RANK chunk (both half-chunks of a rank in one chunk table): the 8 steps of this ring
                "rank_chunk_steps_ms": round(t_rank, 4), "rank_chunk_steps_over_table": round(t_rank / t_tab, 4),
                "rank_chunk_steps_tflops": round(f_share / t_rank / 1e9, 1)})
    return out


def _run_c1(la, torch):
    """Config 1 (the reference's CPU-runnable plumbing case and its acceptance dtype: B=2, H=8, S=1024 as 4 ranks x 256,
    D=64, fp32, causal): every rank's chunk against the chunks it sees, forward alone and forward+backward, on the fp32
    kernels.  The whole config is 2.1e9 flop (forward), microseconds of work: it measures launches, not the matrix pipe,
    so a larger fp32 problem (B=2, H=8, S=4096, one chunk) is timed beside it.  Fractions are of the fp32 MFMA peak."""
    dev = torch.device("cuda:0")
    PEAK32 = 157.3

    def case(B, H, D, S, W):
        sl = S // W
        g = torch.Generator().manual_seed(0)
        q, k, v, do = (torch.randn(B, S, H, D, generator=g).to(dev) for _ in range(4))
        o = torch.empty_like(q)
        lse = torch.empty(W, B, H, sl, dtype=torch.float32, device=dev)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        tabs = []
        for r in range(W):
            order = [(r - s_) % W for s_ in range(W)]
            tabs.append(([k[:, j * sl:(j + 1) * sl] for j in order], [v[:, j * sl:(j + 1) * sl] for j in order],
                         [j * sl for j in order], [dk[:, j * sl:(j + 1) * sl] for j in order], [dv[:, j * sl:(j + 1) * sl] for j in order]))

        def fwd():
            for r in range(W):
                ks, vs, pos, _, _ = tabs[r]
                la.attn_fwd(q[:, r * sl:(r + 1) * sl], ks, vs, pos, r * sl, None, True, out=o[:, r * sl:(r + 1) * sl], lse=lse[r])

        def fwd_bwd():
            fwd()
            dq.zero_(); dk.zero_(); dv.zero_()
            for r in range(W):
                ks, vs, pos, dks, dvs = tabs[r]
                rows = slice(r * sl, (r + 1) * sl)
                d = la.attn_delta(o[:, rows], do[:, rows])
                la.attn_bwd_accumulate(q[:, rows], do[:, rows], lse[r], d, ks, vs, pos, dq[:, rows], dks, dvs, r * sl, None, True)

        def timed(fn, min_s=0.2):
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
            n, t0 = 0, time.perf_counter()
            while time.perf_counter() - t0 < min_s:
                for _ in range(10):
                    fn()
                n += 10
                torch.cuda.synchronize()
            return (time.perf_counter() - t0) / n
        f_fwd = 4.0 * B * H * D * (S * (S + 1) // 2)
        t_f, t_fb = timed(fwd), timed(fwd_bwd)
        plan = la.attn_plan(B, H, H, D, sl, [sl] * W, [j * sl for j in range(W)], (W - 1) * sl, None, True, dtype=torch.float32)
        return {"fwd_us": round(t_f * 1e6, 1), "fwd_tflops": round(f_fwd / t_f / 1e12, 3), "fwd_frac_of_fp32_mfma_peak": round(f_fwd / t_f / 1e12 / PEAK32, 4),
                "fwd_bwd_us": round(t_fb * 1e6, 1), "fwd_bwd_tflops": round(3.5 * f_fwd / t_fb / 1e12, 3),
                "fwd_bwd_frac_of_fp32_mfma_peak": round(3.5 * f_fwd / t_fb / 1e12 / PEAK32, 4), "fwd_kernel": plan["fwd"]["kernel"]}

    return {"what": "fp32 path; config 1 = B=2 H=8 S=1024 (4 ranks x 256) D=64 causal, 4 launches per pass; large = B=2 H=8 S=4096 D=64 causal, one chunk",
            "fp32_mfma_peak_tflops": PEAK32, "config1": case(2, 8, 64, 1024, 4), "large": case(2, 8, 64, 4096, 1)}


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c3", choices=["c2", "c3", "c4", "c5", "s2k", "rope", "mfma_ceiling", "c3_stepwise", "c1", "ref_default"])
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
    la._lib.load()
    torch.cuda.set_device(0)
    if args.workload in ("c3_stepwise", "c1", "ref_default"):
        # side workloads on their own (for profiles): the entry that the default run reports under other_workloads
        fn = {"c3_stepwise": lambda: _run_c3_stepwise(la, torch, args.steps, args.warmup), "c1": lambda: _run_c1(la, torch),
              "ref_default": lambda: _run_ref_default(la, torch)}[args.workload]
        print(json.dumps({"workload": args.workload, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "result": fn()}), flush=True)
        return
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
        torch.cuda.empty_cache()
        others["c3_stepwise"] = _run_c3_stepwise(la, torch, 5, 2)
        torch.cuda.empty_cache()
        others["c1"] = _run_c1(la, torch)
        others["ref_default"] = _run_ref_default(la, torch)
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
