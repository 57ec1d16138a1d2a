"""CPU tests of the host side: the C-ABI library loads and exports what include/ltr_attn.h
declares, argument validation answers without a GPU, and the Ulysses permutation matches the
oracle's restatement of parallel_cp.py:49-96."""
import ctypes
import os
import re

import pytest
import torch

from oracle import ring_attention_oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _lib():
    from lightron_amd import _lib as L
    if not os.path.exists(L.LIB_PATH):
        import lightron_amd.build as b
        b.build()
    return L, L.load()


def _declared(header):
    hdr = open(os.path.join(ROOT, "include", header)).read()
    return set(re.findall(r"^(?:int|const char \*)\s*\*?(ltr_\w+)\(", hdr, flags=re.M))


def _exported(path):
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", path], capture_output=True, text=True, check=True).stdout
    return {ln.split()[-1] for ln in out.splitlines() if " T " in ln and ln.split()[-1].startswith("ltr_")}


def test_header_symbols_exported():
    L, lib = _lib()
    declared = _declared("ltr_attn.h")
    assert declared == set(L.EXPORTS), declared
    for name in declared:
        assert getattr(lib, name) is not None
    # the product library exports the attention path and nothing else
    assert _exported(L.LIB_PATH) == declared
    assert lib.ltr_abi_version() == 8
    assert lib.ltr_strerror(0) == b"ok" and b"aligned" in lib.ltr_strerror(-3)


def test_probe_library_is_separate():
    """The measurement helpers of bench.py live in a library of their own (include/ltr_probe.h)."""
    L, _ = _lib()
    probe = L.load_probe()
    declared = _declared("ltr_probe.h")
    assert declared == set(L.PROBE_EXPORTS) == _exported(L.PROBE_LIB_PATH)
    for name in declared:
        assert getattr(probe, name) is not None
    assert probe.ltr_device_info(None) == -1 and probe.ltr_probe_mfma(None, 0, 1, 0, None) == -1


def test_struct_layout_matches_header():
    # sizes computed from the header's field lists: catches a drifted ctypes mirror
    L, _ = _lib()
    assert ctypes.sizeof(L.KvChunk) == 48
    assert ctypes.sizeof(L.FwdArgs) == 3 * 8 + 4 * 4 + 8 + 4 * 24 + 16 + 8 + 4 * 5 + 4 + 32 * 48 + 3 * 8 + 8 + 24
    assert ctypes.sizeof(L.DeltaArgs) == 3 * 8 + 3 * 4 + 4 + 8 + 2 * 24 + 2 * 4
    assert ctypes.sizeof(L.BwdArgs) == 5 * 8 + 4 * 4 + 8 + 7 * 24 + 16 + 8 + 4 * 4 + 32 * 48 + 8 + 24 + 3 * 8
    assert ctypes.sizeof(L.RopeArgs) == 3 * 8 + 3 * 4 + 4 + 8 + 2 * 24 + 2 * 4
    assert ctypes.sizeof(L.DeviceInfo) == 4 * 4 + 2 * 8 + 64


def _plan(L, lib, D, B, Hq, Hkv, Sq, chunks, flags=0, dtype=None, q_pos0=(0, 0), q_split=None):
    a = L.BwdArgs()
    a.B, a.Hq, a.Hkv, a.D, a.Sq, a.n_chunks = B, Hq, Hkv, D, Sq, len(chunks)
    a.q_pos0[0], a.q_pos0[1], a.q_split = q_pos0[0], q_pos0[1], Sq if q_split is None else q_split
    a.flags, a.io_dtype = flags, L.LTR_BF16 if dtype is None else dtype
    for i, (sk, pos0) in enumerate(chunks):
        a.chunk[i].sk, a.chunk[i].pos0 = sk, pos0
    out = L.AttnPlan()
    rc = lib.ltr_attn_plan(ctypes.byref(a), ctypes.byref(out))
    return rc, out


def test_plan_names_the_kernels_and_follows_the_hints():
    """ltr_attn_plan (host only; 256 compute units without a device) answers with the block sizes the launches would use:
    head dim 128 has one size of each kernel, head dim 64 two, and every LTR_*_ROWS_* / LTR_DKDV_KEYS_* hint forces its size."""
    L, lib = _lib()
    assert ctypes.sizeof(L.AttnPlan) == 6 * 4 + 3 * 8 + 3 * 48
    assert lib.ltr_attn_plan(None, None) == -1
    # config 3, one zig-zag rank share: 16 half-chunks of 2048 keys
    hc = 2048
    rc, pl = _plan(L, lib, 128, 1, 32, 8, 4096, [(hc, i * hc) for i in range(16)], L.LTR_CAUSAL, q_pos0=(0, 15 * hc), q_split=hc)
    assert rc == 0 and pl.compute_units > 0
    assert (pl.fwd_kernel, pl.dq_kernel, pl.dkdv_kernel) == (b"fwd_bf16_kernel<128, 1>", b"bwd_dq_kernel<128, 1>", b"bwd_dkdv_kernel<128, 1>")
    assert (pl.fwd_rows, pl.dq_rows, pl.dkdv_keys) == (256, 256, 128)
    assert pl.dkdv_blocks == 16 * (hc // 128) * 8 and pl.fwd_blocks == pl.dq_blocks
    assert pl.fwd_blocks in (16 * 32, 8 * 32)            # one tile per block, or late + early tile paired
    # head dim 64: both sizes exist; the hints force them, whatever the library would have chosen
    shape = (64, 8, 4, 4, 4096, [(4096, 0)])
    for fl, field, want in ((L.LTR_FWD_ROWS_256, "fwd_rows", 256), (L.LTR_FWD_ROWS_512, "fwd_rows", 512),
                            (L.LTR_DQ_ROWS_256, "dq_rows", 256), (L.LTR_DQ_ROWS_512, "dq_rows", 512),
                            (L.LTR_DKDV_KEYS_128, "dkdv_keys", 128), (L.LTR_DKDV_KEYS_256, "dkdv_keys", 256)):
        rc, pl = _plan(L, lib, *shape, flags=fl)
        assert rc == 0 and getattr(pl, field) == want, (fl, field)
    rc, pl = _plan(L, lib, *shape, flags=L.LTR_DKDV_KEYS_256 | L.LTR_DQ_ROWS_512 | L.LTR_FWD_ROWS_512)
    assert (pl.fwd_kernel, pl.dq_kernel, pl.dkdv_kernel) == (b"fwd_bf16_kernel<64, 2>", b"bwd_dq_kernel<64, 2>", b"bwd_dkdv_kernel<64, 2>")
    assert pl.dkdv_blocks == (4096 // 256) * 8 * 4 and pl.fwd_blocks == (4096 // 512) * 8 * 4
    rc, pl = _plan(L, lib, *shape)                         # config 5's shape: the library's own choice on 256 CUs
    assert rc == 0 and pl.dkdv_keys in (128, 256) and pl.dkdv_blocks == (4096 // pl.dkdv_keys) * 32
    # the wide blocks are bf16, head dim 64 only
    assert _plan(L, lib, 128, 1, 4, 4, 512, [(512, 0)], flags=L.LTR_DKDV_KEYS_256)[0] == -2
    assert _plan(L, lib, 64, 1, 4, 4, 512, [(512, 0)], flags=L.LTR_DQ_ROWS_512, dtype=L.LTR_F32)[0] == -2
    assert _plan(L, lib, 64, 1, 4, 4, 512, [(512, 0)], flags=L.LTR_DQ_ROWS_512 | L.LTR_DQ_ROWS_256)[0] == -1
    assert _plan(L, lib, 96, 1, 4, 4, 512, [(512, 0)])[0] == -2
    rc, pl = _plan(L, lib, 64, 2, 8, 8, 1024, [(256, 0)] * 4, dtype=L.LTR_F32)    # config 1's shape, scalar fp32 kernels
    assert rc == 0 and pl.fwd_kernel == b"fwd_f32_mfma_kernel<64, 2>" and pl.fwd_rows == 64
    assert pl.dq_kernel == b"bwd_dq_f32_mfma_kernel<64, 2>" and pl.dq_rows == 64
    assert pl.dkdv_kernel == b"bwd_dkdv_f32_mfma_kernel<64>" and pl.dkdv_keys == 128 and pl.dkdv_blocks == 4 * 2 * 16
    rc, pl = _plan(L, lib, 64, 2, 8, 8, 1024, [(256, 0)] * 4, dtype=L.LTR_F32, flags=L.LTR_FWD_F32_SCALAR | L.LTR_BWD_F32_SCALAR)
    assert rc == 0 and pl.fwd_kernel == b"fwd_f32_kernel<64>" and pl.fwd_rows == 64
    assert pl.dq_kernel == b"bwd_dq_f32_kernel<64>" and pl.dkdv_keys == 64 and pl.dkdv_blocks == 4 * 4 * 16
    assert _plan(L, lib, 64, 1, 4, 4, 512, [(512, 0)], flags=L.LTR_BWD_F32_SCALAR)[0] == -2      # fp32 only, as in the launches


def test_validation_without_gpu():
    L, lib = _lib()
    assert lib.ltr_attn_fwd(None, None) == -1
    a = L.FwdArgs()
    assert lib.ltr_attn_fwd(ctypes.byref(a), None) == -1            # null pointers
    a.q = a.o = a.lse = 4096
    a.B, a.Hq, a.Hkv, a.D, a.Sq, a.n_chunks = 1, 4, 3, 128, 16, 1
    assert lib.ltr_attn_fwd(ctypes.byref(a), None) == -1            # Hq % Hkv
    a.Hkv, a.D = 2, 96
    assert lib.ltr_attn_fwd(ctypes.byref(a), None) == -2            # head dim
    a.D, a.n_chunks = 128, 33
    assert lib.ltr_attn_fwd(ctypes.byref(a), None) == -1            # too many chunks
    a.n_chunks, a.q, a.q_split = 1, 4100, 16
    assert lib.ltr_attn_fwd(ctypes.byref(a), None) == -3            # misaligned q
    a.q = 4096
    a.q_stride[1] = 4                                               # 8-byte row stride in bf16
    assert lib.ltr_attn_fwd(ctypes.byref(a), None) == -3
    assert lib.ltr_attn_bwd(None, None) == -1 and lib.ltr_attn_bwd_delta(None, None) == -1
    assert lib.ltr_cast_f32_to_bf16(None, None, 4, None) == -1
    assert lib.ltr_cast_f32_to_bf16(4096, 4096, 0, None) == 0       # empty input is a no-op
    assert lib.ltr_rope_apply(None, None) == -1
    r = L.RopeArgs()
    assert lib.ltr_rope_apply(ctypes.byref(r), None) == -1          # null pointers
    r.x = r.out = r.freqs = 4096
    r.B, r.H, r.D, r.S = 1, 2, 12, 4
    assert lib.ltr_rope_apply(ctypes.byref(r), None) == -2          # head dim not a multiple of 8
    r.D, r.io_dtype = 16, 7
    assert lib.ltr_rope_apply(ctypes.byref(r), None) == -2          # dtype
    r.io_dtype, r.x = 0, 4100
    assert lib.ltr_rope_apply(ctypes.byref(r), None) == -3          # misaligned x
    r.x = 4096
    r.x_stride[1] = 4
    assert lib.ltr_rope_apply(ctypes.byref(r), None) == -3          # 8-byte row stride in bf16
    r.x_stride[1], r.S = 32, 0
    assert lib.ltr_rope_apply(ctypes.byref(r), None) == 0           # empty input is a no-op


def test_no_alloc_entry_point_validation_without_gpu():
    L, lib = _lib()
    assert lib.ltr_attn_bwd_noalloc(None, None) == -1
    a = L.BwdArgs()
    a.q = a.d_o = a.lse = a.dq = a.o = 4096
    a.B, a.Hq, a.Hkv, a.D, a.n_chunks, a.io_dtype = 1, 32, 8, 128, 1, L.LTR_BF16
    a.Sq = L.LTR_NOALLOC_MAX_ROWS // 32 + 1
    assert lib.ltr_attn_bwd_noalloc(ctypes.byref(a), None) == -6      # more DELTA rows than the fixed scratch holds
    assert b"scratch" in lib.ltr_strerror(-6)
    a.Sq, a.flags = 64, L.LTR_NO_DQ
    assert lib.ltr_attn_bwd_noalloc(ctypes.byref(a), None) == -1      # the dQ kernel is the one that fills DELTA
    a.flags, a.io_dtype = 0, L.LTR_F32
    assert lib.ltr_attn_bwd_noalloc(ctypes.byref(a), None) == -2      # bf16 only


def test_fused_rope_validation_without_gpu():
    L, lib = _lib()
    a = L.FwdArgs()
    a.q = a.o = a.lse = 4096
    a.B, a.Hq, a.Hkv, a.D, a.Sq, a.n_chunks, a.q_split = 1, 4, 2, 128, 64, 1, 64
    a.io_dtype = a.o_dtype = L.LTR_BF16
    a.flags = L.LTR_ROPE_Q
    assert lib.ltr_attn_fwd(ctypes.byref(a), None) == -1            # no table
    a.rope_freqs, a.rope_pos0, a.rope_len = 4096, 0, 32
    assert lib.ltr_attn_fwd(ctypes.byref(a), None) == -1            # table ends before the last row's position
    a.rope_len = 64
    a.q_pos0[0] = a.q_pos0[1] = 10
    assert lib.ltr_attn_fwd(ctypes.byref(a), None) == -1            # rows at positions 10 .. 73
    a.rope_pos0 = 10
    a.rope_freqs = 4100
    assert lib.ltr_attn_fwd(ctypes.byref(a), None) == -3            # misaligned table
    a.rope_freqs, a.io_dtype, a.o_dtype = 4096, L.LTR_F32, L.LTR_F32
    assert lib.ltr_attn_fwd(ctypes.byref(a), None) == -2            # bf16 only
    b = L.BwdArgs()
    b.q = b.d_o = b.lse = b.delta = b.dq = 4096
    b.B, b.Hq, b.Hkv, b.D, b.Sq, b.n_chunks, b.q_split = 1, 4, 2, 128, 64, 1, 64
    b.io_dtype = L.LTR_BF16
    b.flags = L.LTR_ROPE_DQ | L.LTR_NO_DQ
    b.rope_freqs, b.rope_len = 4096, 64
    assert lib.ltr_attn_bwd(ctypes.byref(b), None) == -1            # the rotation lives in the dQ kernel's epilogue


def test_bench_traffic_figure_is_tied_to_the_kernel_source(tmp_path, monkeypatch):
    """bench.py takes roofline.traffic from the counter profile only while the kernel source still has the hash the
    profile names: a changed source must give None (a stale figure is never reported)."""
    import hashlib
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_mod", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    src = tmp_path / "k.hip"
    src.write_text("kernel text")
    prof = tmp_path / "counters.md"
    digest = hashlib.sha256(src.read_bytes()).hexdigest()
    prof.write_text("x\nkernel-source-sha256: %s\ntraffic-bytes-per-launch bwd_dkdv_kernel<128, 1>: 1.2988e+09\n" % digest)
    monkeypatch.setattr(bench, "KERNEL_SOURCE", str(src))
    monkeypatch.setattr(bench, "COUNTER_PROFILE", str(prof))
    val, why = bench._measured_traffic("bwd_dkdv_kernel<128, 1>")
    assert val == 1.2988e9 and digest[:12] in why
    assert bench._measured_traffic("fwd_bf16_kernel<128, 2>")[0] is None   # no line for that kernel
    src.write_text("kernel text, edited")
    val, why = bench._measured_traffic("bwd_dkdv_kernel<128, 1>")
    assert val is None and "stale" in why
    # the committed profile and the committed source: either in step (a number) or flagged, never an exception
    monkeypatch.undo()
    val, why = bench._measured_traffic("bwd_dkdv_kernel<128, 1>")
    assert (val is None) or val > 0


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode != 0 and "ONE GPU" in (res.stderr + res.stdout)
    env = dict(os.environ, WORLD_SIZE="2")
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")], capture_output=True, text=True, env=env)
    assert res.returncode != 0 and "ONE GPU" in (res.stderr + res.stdout)


def test_missing_library_fails_loudly(monkeypatch):
    from lightron_amd import _lib as L
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "LIB_PATH", "/nonexistent/libltr_attn.so")
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        L.load()


def test_cpu_tensors_are_refused():
    import lightron_amd as la
    q = torch.zeros(1, 8, 2, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        la.attn_fwd(q, [q], [q], [0])


@pytest.mark.parametrize("W", [1, 2, 4])
def test_seq_all_to_all_matches_oracle_and_backward(W):
    import lightron_amd as la
    B, Sl, H, D = 2, 3, 8, 4
    g = torch.Generator().manual_seed(3)
    x = torch.randn(W, B, Sl, H, D, generator=g, requires_grad=True)
    grp = la.LocalCPGroup(W)
    y = la._all_to_all(x if W > 1 else x[0], 2, 1, grp)
    ref = orc.seq_all_to_all([x[r].detach() for r in range(W)], 2, 1)
    if W == 1:
        assert y is x[0] or torch.equal(y, x[0])
        return
    for r in range(W):
        assert torch.equal(y[r], ref[r])
    back = la._all_to_all(y, 1, 2, grp)
    assert torch.equal(back, x)
    # backward = the exchange with the two dims swapped (parallel_cp.py:85-93)
    gy = torch.randn(y.shape, generator=g)
    y.backward(gy)
    gref = orc.seq_all_to_all([gy[r] for r in range(W)], 1, 2)
    for r in range(W):
        assert torch.equal(x.grad[r], gref[r])


def test_seq_all_to_all_refuses_indivisible_and_real_groups():
    import lightron_amd as la
    x = torch.zeros(4, 1, 2, 6, 2)
    with pytest.raises(AssertionError):
        la._all_to_all(x, 2, 1, la.LocalCPGroup(4))
    assert torch.equal(la._all_to_all(x, 2, 1, None), x)
    with pytest.raises(NotImplementedError):
        la._all_to_all(x, 2, 1, object())


def test_ring_descriptor_order_and_positions():
    from lightron_amd.ring_attention import LocalRing, _chunk_table
    ring = LocalRing(2, 4, kv=[(torch.zeros(1, 8, 1, 4), torch.zeros(1, 8, 1, 4))] * 4, layout="zigzag")
    assert ring.order() == orc.ring_order(2, 4) == [2, 1, 0, 3]
    ks, vs, pos, _ = _chunk_table(ring, None, None, 8)
    exp = []
    for j in ring.order():
        p = orc.zigzag_positions(j, 4, 32)
        exp += [int(p[0]), int(p[4])]
    assert pos == exp and all(k.shape[1] == 4 for k in ks)
    with pytest.raises(NotImplementedError):
        import lightron_amd as la
        la.ring_attention_kernel(torch.zeros(1, 8, 1, 64), None, None, object(), None)


def test_rope_helpers_match_oracle():
    import lightron_amd as la
    fc = la.precompute_freqs_cis(16, 32)
    assert (fc - orc.precompute_freqs_cis(16, 32)).abs().max() < 1e-6
    g = torch.Generator().manual_seed(5)
    q, k = torch.randn(2, 32, 3, 16, generator=g), torch.randn(2, 32, 3, 16, generator=g)
    with pytest.raises(RuntimeError, match="GPU tensors"):      # no host path: the rotation itself is checked on the GPU
        la.apply_rotary_emb(q, k, fc)
    tab = la.rope_table(fc)
    assert tab.shape == (32, 8, 2) and tab.dtype == torch.float32
    assert torch.equal(tab[..., 0], fc.real) and torch.equal(tab[..., 1], fc.imag)
    with pytest.raises(AssertionError):
        la.layers.reshape_for_broadcast(fc[:16], torch.view_as_complex(q.reshape(2, 32, 3, 8, 2)))
