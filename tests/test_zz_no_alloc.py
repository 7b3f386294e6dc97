"""olmax_attn_bwd_noalloc (the entry point for callers that cannot allocate: its delta scratch is
a device array inside the library) against olmax_attn_bwd with a caller-provided workspace, through
the C ABI: same kernels, so the three gradients must be bit-identical.  Two calls in a row, the
second on a smaller input, so that whatever the first call left in the shared array is stale data
for the second; then the size and alignment limits, which must be refused on the host."""
import ctypes
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _inputs(B, S, H, KH, seed):
    g = torch.Generator().manual_seed(seed)
    mk = lambda cols: torch.randn(B * S, cols, generator=g).to(BF).cuda()
    return mk(H * 128), mk(KH * 128), mk(KH * 128), mk(H * 128)


def _noalloc(L, q, k, v, o, lse, do, B, S, H, KH, window, softcap, D=128):
    from olmax_amd._lib import f32, i32, i64, ptr, stream_ptr
    dq = torch.empty(B * S, H * D, device="cuda", dtype=BF)
    dk = torch.empty(B * S, KH * D, device="cuda", dtype=BF)
    dv = torch.empty(B * S, KH * D, device="cuda", dtype=BF)
    rc = L.olmax_attn_bwd_noalloc(stream_ptr(), ptr(q), ptr(k), ptr(v), ptr(o), ptr(lse), ptr(do), ptr(dq), ptr(dk), ptr(dv),
                                  i32(B), i32(S), i32(H), i32(KH), i32(D), i64(q.stride(0)), i64(k.stride(0)), i64(v.stride(0)),
                                  i64(o.stride(0)), i64(do.stride(0)), i64(dq.stride(0)), i64(dk.stride(0)), i64(dv.stride(0)),
                                  i32(-1 if window is None else window), f32(softcap))
    return rc, dq, dk, dv


def test_attn_bwd_noalloc_equals_attn_bwd_on_two_calls_in_a_row():
    from olmax_amd import _lib, ops
    L = _lib.load()
    L.olmax_attn_bwd_noalloc_max_rows.restype = ctypes.c_int64
    assert L.olmax_attn_bwd_noalloc_max_rows() == 1 << 20
    for (B, S, H, KH, window, softcap, seed) in [(2, 1024, 4, 2, None, 0.0, 1), (1, 328, 2, 1, 100, 30.0, 2)]:
        print(f"[case] attn_bwd_noalloc B{B} S{S} H{H} KH{KH} w{window} cap{softcap}", flush=True)
        sys.stdout.flush()
        q, k, v, do = _inputs(B, S, H, KH, seed)
        o, lse = ops.attn_fwd(q, k, v, B=B, S=S, H=H, KH=KH, D=128, window=window, softcap=softcap)
        want = ops.attn_bwd(q, k, v, o, lse, do, B=B, S=S, H=H, KH=KH, D=128, window=window, softcap=softcap)
        rc, dq, dk, dv = _noalloc(L, q, k, v, o, lse, do, B, S, H, KH, window, softcap)
        assert rc == 0, L.olmax_last_error_string()
        torch.cuda.synchronize()
        for name, a, b in zip(("dq", "dk", "dv"), (dq, dk, dv), want):
            assert torch.equal(a, b), name
        assert dq.float().abs().sum().item() > 0


def test_attn_bwd_noalloc_replays_from_a_graph_after_set_up():
    """The entry point recorded into a HIP graph (its reason for being): set-up
    (olmax_attn_bwd_noalloc_init, which resolves the scratch address for the device) happens
    before the capture; three replays with fresh inputs copied into the captured buffers, eager
    work and a synchronisation between them, each checked against olmax_attn_bwd."""
    from olmax_amd import _lib, ops
    L = _lib.load()
    assert L.olmax_attn_bwd_noalloc_init() == 0, L.olmax_last_error_string()
    B, S, H, KH = 1, 512, 4, 2
    print(f"[case] attn_bwd_noalloc under graph capture B{B} S{S} H{H} KH{KH}", flush=True)
    q, k, v, do = _inputs(B, S, H, KH, 10)
    o, lse = ops.attn_fwd(q, k, v, B=B, S=S, H=H, KH=KH, D=128)
    dq = torch.empty(B * S, H * 128, device="cuda", dtype=BF)
    dk = torch.empty(B * S, KH * 128, device="cuda", dtype=BF)
    dv = torch.empty(B * S, KH * 128, device="cuda", dtype=BF)
    from olmax_amd._lib import f32, i32, i64, ptr, stream_ptr

    def record():
        return L.olmax_attn_bwd_noalloc(stream_ptr(), ptr(q), ptr(k), ptr(v), ptr(o), ptr(lse), ptr(do), ptr(dq), ptr(dk), ptr(dv),
                                        i32(B), i32(S), i32(H), i32(KH), i32(128), i64(q.stride(0)), i64(k.stride(0)), i64(v.stride(0)),
                                        i64(o.stride(0)), i64(do.stride(0)), i64(dq.stride(0)), i64(dk.stride(0)), i64(dv.stride(0)),
                                        i32(-1), f32(0.0))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        assert record() == 0, L.olmax_last_error_string()
    for rep in range(3):
        q2, k2, v2, do2 = _inputs(B, S, H, KH, 20 + rep)
        o2, lse2 = ops.attn_fwd(q2, k2, v2, B=B, S=S, H=H, KH=KH, D=128)
        want = ops.attn_bwd(q2, k2, v2, o2, lse2, do2, B=B, S=S, H=H, KH=KH, D=128)
        for dst, src in ((q, q2), (k, k2), (v, v2), (do, do2), (o, o2), (lse, lse2)):
            dst.copy_(src)
        dq.zero_(); dk.zero_(); dv.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("dq", "dk", "dv"), (dq, dk, dv), want):
            assert torch.equal(a, b), (rep, name)


def test_attn_bwd_noalloc_refuses_what_it_cannot_hold():
    from olmax_amd import _lib, ops
    L = _lib.load()
    B, S, H, KH = 1, 64, 2, 1
    q, k, v, do = _inputs(B, S, H, KH, 3)
    o, lse = ops.attn_fwd(q, k, v, B=B, S=S, H=H, KH=KH, D=128)
    # beyond the built-in scratch: refused on the host before any launch (the shapes are only claimed)
    rc, *_ = _noalloc(L, q, k, v, o, lse, do, 65, 8192, H, KH, None, 0.0)  # 65 * 2 * 8192 > 2^20
    assert rc == -5 and b"exceeds the built-in scratch" in L.olmax_last_error_string()
    # not the MFMA path (unaligned view): refused, the caller is pointed at olmax_attn_bwd
    wide = torch.zeros(B * S, H * 128 + 8, device="cuda", dtype=BF)
    rc, *_ = _noalloc(L, wide[:, 4:4 + H * 128], k, v, o, lse, do, B, S, H, KH, None, 0.0)
    assert rc == -3 and b"olmax_attn_bwd" in L.olmax_last_error_string()
    rc, *_ = _noalloc(L, q, k, v, o, lse, do, B, S, 4, 2, None, 0.0, D=64)
    assert rc == -3
