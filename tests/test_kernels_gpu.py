"""GPU parity tests: every HIP entry point, called through the C ABI, against the CPU oracle
on the same seeded inputs.  Tolerances follow the stated gates: activations within 1e-2
relative (bf16), gradient cosine similarity >= 0.999; integer/index work bit-exact."""
import math
import sys

import pytest
import torch

from oracle import ref

pytestmark = pytest.mark.gpu

BF = torch.bfloat16
rt = ref.bf16_round


def _ops():
    from olmax_amd import ops
    return ops


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def relerr(got: torch.Tensor, want: torch.Tensor) -> float:
    got, want = got.double().cpu(), want.double().cpu()
    return ((got - want).norm() / (want.norm() + 1e-30)).item()


def maxrel(got, want) -> float:
    got, want = got.double().cpu(), want.double().cpu()
    return ((got - want).abs().max() / (want.abs().max() + 1e-30)).item()


def cosine(a, b) -> float:
    a, b = a.double().cpu().flatten(), b.double().cpu().flatten()
    return (a @ b / (a.norm() * b.norm() + 1e-30)).item()


def bfr(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(BF)


def check_close(got, want, name, tol=1e-2, cos=0.9999):
    e, c = relerr(got, want), cosine(got, want)
    assert e < tol and c > cos, f"{name}: relerr {e:.3e} cosine {c:.6f}"


@pytest.mark.parametrize("M,N,K", [(256, 512, 128), (384, 128, 192), (1024, 2048, 512), (50, 36, 20), (129, 257, 65)])
@pytest.mark.parametrize("al,bl", [(0, 0), (0, 1), (1, 1), (1, 0)])
def test_gemm_layouts(M, N, K, al, bl):
    ops = _ops()
    say(f"gemm M{M} N{N} K{K} a{al} b{bl}")
    a = bfr(*((M, K) if al == 0 else (K, M)), seed=1)
    b = bfr(*((N, K) if bl == 0 else (K, N)), seed=2)
    r = bfr(M, N, seed=3)
    af = a.double() if al == 0 else a.double().t()
    bf_ = b.double() if bl == 0 else b.double().t()
    want = af @ bf_.t()
    got = ops.gemm(a.cuda(), b.cuda(), a_layout=al, b_layout=bl)
    assert maxrel(got, want) < 6e-3
    plain = got
    got = ops.gemm(a.cuda(), b.cuda(), a_layout=al, b_layout=bl, residual=r.cuda(), out_f32=True)
    assert maxrel(got, want + r.double()) < 1e-5
    got = ops.gemm(a.cuda(), b.cuda(), a_layout=al, b_layout=bl, residual=r.cuda())
    assert torch.equal(got, (plain.float() + r.cuda().float()).to(BF))  # bf16(bf16(A B^T) + R), every tile size


def test_gemm_brute_force_tiny_and_strided():
    ops = _ops()
    say("gemm tiny brute force + strided views")
    a = bfr(3, 5, seed=4); b = bfr(4, 5, seed=5)
    got = ops.gemm(a.cuda(), b.cuda(), out_f32=True).cpu()
    for i in range(3):
        for j in range(4):
            assert abs(got[i, j].item() - sum(float(a[i, k]) * float(b[j, k]) for k in range(5))) < 1e-5
    # row-strided operands (column slices of wider buffers), MFMA path
    big_a = bfr(256, 512, seed=6).cuda(); big_b = bfr(256, 384, seed=7).cuda()
    av, bv = big_a[:, 128:384], big_b[:, 64:320]
    got = ops.gemm(av, bv)
    assert maxrel(got, av.double().cpu() @ bv.double().cpu().t()) < 6e-3


@pytest.mark.parametrize("al,bl", [(0, 0), (0, 1), (1, 1), (1, 0)])
@pytest.mark.parametrize("M,N,K", [(2048, 4096, 192), (2048, 4096, 256), (4096, 4352, 64), (4096, 8448, 256), (4096, 12288, 384)])
def test_gemm_256_tiles_row_strided_operands(M, N, K, al, bl):
    """The 256x256-tile kernel (>= 128 tiles) with every operand a column slice of a wider buffer
    (leading dimensions that are not the row length, 16-byte aligned offsets), odd and even k-tile
    counts, a strided residual and a strided output; the 272-tile case is cut into whole rounds
    plus a remainder; the 528- and 768-tile cases have more tiles than the GPU has CUs (two and
    three rounds of workgroups).  Against a float64 product of the same bf16 values."""
    ops = _ops()
    say(f"gemm 256-tile strided M{M} N{N} K{K} a{al} b{bl}")
    ar, ac = (M, K) if al == 0 else (K, M)
    br, bc = (N, K) if bl == 0 else (K, N)
    big_a = bfr(ar, ac + 72, seed=11).cuda(); big_b = bfr(br, bc + 40, seed=12, scale=0.05).cuda()
    av, bv = big_a[:, 8:8 + ac], big_b[:, 24:24 + bc]
    big_r = bfr(M, N + 16, seed=13).cuda(); rv = big_r[:, 8:8 + N]
    af = av.double() if al == 0 else av.double().t()
    bf_ = bv.double() if bl == 0 else bv.double().t()
    want = (af @ bf_.t()).cpu()
    got = ops.gemm(av, bv, a_layout=al, b_layout=bl)
    assert maxrel(got, want) < 6e-3
    out = torch.zeros(M, N + 24, device="cuda", dtype=BF)
    ops.gemm(av, bv, a_layout=al, b_layout=bl, residual=rv, out=out[:, 16:16 + N])
    assert maxrel(out[:, 16:16 + N], want + rv.double().cpu()) < 6e-3
    # the residual joins the ROUNDED product, like the reference's `x + linear(...)` on bf16 arrays:
    # bit-equal to the plain product plus the residual, rounded once more
    assert torch.equal(out[:, 16:16 + N], (got.float() + rv.float()).to(BF))
    assert not out[:, :16].any() and not out[:, 16 + N:].any()  # nothing written outside the view


@pytest.mark.parametrize("M,N,K,al,bl", [(8192, 3072, 256, 0, 0), (2048, 5120, 192, 0, 1), (4096, 2048, 320, 1, 1),
                                          (2048 + 512, 2048 + 768, 128, 0, 0), (6144, 11008, 64, 1, 1)])
def test_gemm_tile_order_does_not_change_results(M, N, K, al, bl):
    """Which tile a workgroup takes is a scheduling choice (one run of tiles per XCD, or windows of
    8 x 4 tiles dealt so that the XCDs cover 1, 2, 4 or 8 strips of tile rows together, on grids
    that divide into windows and on grids that need padded windows and surplus workgroups): every
    order must cover every tile exactly once, so the products are bit-identical."""
    ops = _ops()
    from olmax_amd import _lib
    L = _lib.load()
    say(f"gemm tile orders M{M} N{N} K{K} a{al} b{bl}")
    a = bfr(*((M, K) if al == 0 else (K, M)), seed=21).cuda()
    b = bfr(*((N, K) if bl == 0 else (K, N)), seed=22).cuda()
    r = bfr(M, N, seed=23).cuda()
    outs = []
    try:
        for order in (-1, 0, 1, 2, 4, 8):
            L.olmax_gemm_set_order(order)
            out = torch.full((M, N), float("nan"), device="cuda", dtype=BF)
            ops.gemm(a, b, a_layout=al, b_layout=bl, residual=r, out=out)
            outs.append(out)
    finally:
        L.olmax_gemm_set_order(0)
    torch.cuda.synchronize()
    assert not torch.isnan(outs[0].float()).any()
    for o in outs[1:]:
        assert torch.equal(o, outs[0])
    af = a.double() if al == 0 else a.double().t()
    bf_ = b.double() if bl == 0 else b.double().t()
    assert maxrel(outs[0], (af @ bf_.t() + r.double()).cpu()) < 6e-3


def test_gemm_rejects_bad_arguments():
    ops = _ops()
    from olmax_amd._lib import OlmaxHipError
    with pytest.raises(AssertionError):
        ops.gemm(bfr(4, 5).cuda(), bfr(4, 6).cuda())
    with pytest.raises(OlmaxHipError):
        ops.gemm(bfr(4, 5), bfr(4, 5))  # CPU tensors: no fallback


@pytest.mark.parametrize("rows,d", [(64, 4096), (37, 256), (130, 128), (16, 5376), (9, 4608), (5, 100), (3, 16), (4100, 4096), (2500, 128),
                                    (300, 3080), (1030, 2056), (77, 1032), (519, 2048), (40, 1024), (1025, 8192), (33, 6152), (7, 264)])
def test_rmsnorm(rows, d):
    ops = _ops()
    say(f"rmsnorm rows{rows} d{d}")
    x = bfr(rows, d, seed=1); w = (1 + 0.1 * torch.randn(d, generator=torch.Generator().manual_seed(2))).to(BF)
    dy = bfr(rows, d, seed=3); dres = bfr(rows, d, seed=4)
    y = ops.rms_norm_fwd(x.cuda(), w.cuda(), 1e-6)
    want = ref.rms_norm_fwd(x.double(), w.double(), 1e-6)
    assert maxrel(y, want) < 1e-2
    dx, dw = ops.rms_norm_bwd(x.cuda(), w.cuda(), dy.cuda(), 1e-6)
    wdx, wdw = ref.rms_norm_bwd(x.double(), w.double(), dy.double(), 1e-6)
    check_close(dx, wdx, "dx"); check_close(dw, wdw, "dw")
    # accumulation into a given dw
    acc = torch.full((d,), 0.5, device="cuda")
    ops.rms_norm_bwd(x.cuda(), w.cuda(), dy.cuda(), 1e-6, dw=acc)
    check_close(acc - 0.5, wdw, "dw accumulated", tol=2e-2)
    dx2, _ = ops.rms_norm_bwd(x.cuda(), w.cuda(), dy.cuda(), 1e-6, dres=dres.cuda())
    check_close(dx2, wdx + dres.double(), "dx+dres")
    # no weight
    y0 = ops.rms_norm_fwd(x.cuda(), None, 1e-6)
    assert maxrel(y0, ref.rms_norm_fwd(x.double(), None, 1e-6)) < 1e-2


def test_rmsnorm_empty_and_strided():
    ops = _ops()
    say("rmsnorm empty + strided")
    x = torch.empty(0, 128, dtype=BF).cuda()
    assert ops.rms_norm_fwd(x, None, 1e-6).shape == (0, 128)
    big = bfr(32, 1024, seed=5).cuda()
    v = big[:, 256:768]
    y = ops.rms_norm_fwd(v, None, 1e-5)
    assert maxrel(y, ref.rms_norm_fwd(v.double().cpu(), None, 1e-5)) < 1e-2


@pytest.mark.parametrize("S,D,theta", [(4096, 128, 500000.0), (4096, 128, 10000.0), (4096, 128, 1e6), (512, 64, 10000.0), (77, 16, 3.5)])
def test_rope_tables_follow_the_reference_arithmetic(S, D, theta):
    """olmax_rope_tables against (a) the exact closed form cos/sin(p * theta^(-2i/D)) in float64 and
    (b) the oracle's fp32 table (torch-CPU arithmetic in the reference's order of operations,
    src/olmax/nn/rope.py:127-133).  Both comparisons are by tolerance: the kernel and the oracle are
    two independent fp32 implementations (different powf / cosf), and an fp32 angle is only good
    to a few ulp: |d angle| <= 4 * 2^-23 * angle (pow, reciprocal, product)."""
    ops = _ops()
    say(f"rope tables S{S} D{D} theta{theta}")
    cos, sin = ops.rope_tables(S, D, theta, "cuda")
    assert cos.shape == (S, D // 2) and cos.dtype == torch.float32
    cos, sin = cos.cpu().double(), sin.cpu().double()
    p = torch.arange(S, dtype=torch.float64)[:, None]
    i = torch.arange(D // 2, dtype=torch.float64)[None, :]
    ang = p * theta ** (-2.0 * i / D)
    tol = 4 * 2.0 ** -23 * ang + 2.0 ** -22
    assert ((cos - torch.cos(ang)).abs() <= tol).all() and ((sin - torch.sin(ang)).abs() <= tol).all()
    rc, rs = ref.rope_tables(S, D, theta)
    assert ((cos - rc.double()).abs() <= 2 * tol).all() and ((sin - rs.double()).abs() <= 2 * tol).all()
    # positions are exact integers: frequency 0 (inv_freq == 1) must see the angle p itself
    assert ((cos[:, 0] - torch.cos(p[:, 0])).abs() <= 2.0 ** -22).all()
    assert torch.equal(cos[0], torch.ones(D // 2, dtype=torch.float64)) and torch.equal(sin[0], torch.zeros(D // 2, dtype=torch.float64))


@pytest.mark.parametrize("D,heads,norm", [(128, 4, False), (128, 3, True), (64, 4, False), (16, 2, True)])
def test_qk_rope(D, heads, norm):
    ops = _ops()
    say(f"qk_rope D{D} heads{heads} norm{norm}")
    B, S = 2, 24
    x = bfr(B * S, heads * D, seed=1); dy = bfr(B * S, heads * D, seed=2)
    w = (1 + 0.1 * torch.randn(D, generator=torch.Generator().manual_seed(3))).to(BF) if norm else None
    cos, sin = ops.rope_tables(S, D, 500000.0, "cuda")
    rc, rs = cos.cpu(), sin.cpu()  # the same table feeds kernel and oracle: this test is about the rotation
    y = ops.qk_rope_fwd(x.cuda(), cos, sin, heads=heads, head_dim=D, seq_len=S, w=None if w is None else w.cuda())
    x4 = x.double().reshape(B, S, heads, D)
    xn = rt(ref.rms_norm_fwd(x4, w.double(), 1e-6)) if norm else x4
    want = ref.rope_fwd(xn, rc.double(), rs.double()).reshape(B * S, heads * D)
    assert maxrel(y, want) < 1e-2
    dx, dw = ops.qk_rope_bwd(dy.cuda(), cos, sin, heads=heads, head_dim=D, seq_len=S,
                             x=x.cuda() if norm else None, w=None if w is None else w.cuda())
    g = ref.rope_bwd(dy.double().reshape(B, S, heads, D), rc.double(), rs.double())
    if norm:
        g, wdw = ref.rms_norm_bwd(x4, w.double(), rt(g), 1e-6)
        check_close(dw, wdw, "dw")
    check_close(dx, g.reshape(B * S, heads * D), "dx")


def test_qk_rope_inplace_on_strided_qkv():
    ops = _ops()
    say("qk_rope in place on a fused qkv buffer")
    B, S, H, D = 1, 16, 2, 128
    qkv = bfr(B * S, 3 * H * D, seed=7).cuda()
    orig = qkv.clone()
    cos, sin = ops.rope_tables(S, D, 1e4, "cuda")
    qv = qkv[:, : H * D]
    ops.qk_rope_fwd(qv, cos, sin, heads=H, head_dim=D, seq_len=S, out=qv)
    rc, rs = cos.cpu(), sin.cpu()
    want = ref.rope_fwd(orig[:, : H * D].double().cpu().reshape(B, S, H, D), rc.double(), rs.double()).reshape(B * S, H * D)
    assert maxrel(qkv[:, : H * D], want) < 1e-2
    assert torch.equal(qkv[:, H * D:], orig[:, H * D:])  # k, v untouched


@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("T,F", [(64, 1024), (7, 24), (5, 11)])
def test_glu(act, T, F):
    ops = _ops()
    say(f"glu {act} T{T} F{F}")
    gu = bfr(T, 2 * F, seed=1, scale=2.0); dh = bfr(T, F, seed=2)
    g, u = gu[:, :F], gu[:, F:]
    gc = gu.cuda()
    out = ops.glu_fwd(gc[:, :F], gc[:, F:], act)
    assert maxrel(out, ref.glu_fwd(g.double(), u.double(), act, rt)) < 1e-2
    dg, du = ops.glu_bwd(gc[:, :F], gc[:, F:], dh.cuda(), act)
    wg, wu = ref.glu_bwd(g.double(), u.double(), dh.double(), act)
    check_close(dg, wg, "dgate"); check_close(du, wu, "dup")


@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("T,F,d", [(2048, 2048, 256), (4096, 1024, 128), (96, 40, 24)])
def test_gated_mlp_in_fused_epilogue(act, T, F, d):
    """The GEMM with the GLU epilogue must equal GEMM + glu_fwd bit for bit (same tile, same
    roundings), match the oracle, and not need the gate|up output on fused shapes."""
    ops = _ops()
    say(f"gated_mlp_in {act} T{T} F{F} d{d}")
    x = bfr(T, d, seed=1); w = bfr(2 * F, d, seed=2, scale=d ** -0.5)
    xc, wc = x.cuda(), w.cuda()
    gu_plain = ops.gemm(xc, wc)
    act_plain = ops.glu_fwd(gu_plain[:, :F], gu_plain[:, F:], act)
    act_fused, gu_fused = ops.gated_mlp_in(xc, wc, act)
    assert torch.equal(gu_fused, gu_plain) and torch.equal(act_fused, act_plain)
    fits = T % 256 == 0 and F % 128 == 0 and d % 64 == 0 and (T // 256) * (F // 128) >= 128
    act_only, none = ops.gated_mlp_in(xc, wc, act, save_gate_up=False)
    assert torch.equal(act_only, act_plain) and ((none is None) == fits)
    if T * F * d <= 2 ** 31:
        gu_want = ref.linear_fwd(x.double(), w.double(), rt)
        want = ref.glu_fwd(gu_want[:, :F], gu_want[:, F:], act, rt)
        assert maxrel(act_fused, want) < 2e-2


@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("T,F,d", [(2048, 2048, 256), (4096, 1024, 128), (8192, 5504, 192), (96, 40, 24)])
def test_gated_mlp_in_backward_form(act, T, F, d):
    """The gated projection in its backward form (gate | up recomputed in the accumulators, the GLU
    backward in the epilogue) must equal the forward-form GEMM followed by glu_bwd bit for bit: the
    activation output and d gate | d up; odd shapes take the unfused path inside the call.  Against
    the oracle on the shapes it can hold."""
    ops = _ops()
    say(f"gated_mlp_in backward form {act} T{T} F{F} d{d}")
    x = bfr(T, d, seed=1); w = bfr(2 * F, d, seed=2, scale=d ** -0.5); dact = bfr(T, F, seed=3)
    xc, wc, dc = x.cuda(), w.cuda(), dact.cuda()
    act_plain, gu = ops.gated_mlp_in(xc, wc, act)
    dg, du = ops.glu_bwd(gu[:, :F], gu[:, F:], dc, act)
    act_b, dgu = ops.gated_mlp_in_bwd(xc, wc, dc, act)
    assert torch.equal(act_b, act_plain)
    assert torch.equal(dgu[:, :F], dg) and torch.equal(dgu[:, F:], du)
    if T * F * d <= 2 ** 31:
        gu_want = ref.linear_fwd(x.double(), w.double(), rt)
        wg, wu = ref.glu_bwd(gu_want[:, :F], gu_want[:, F:], dact.double(), act)
        check_close(dgu[:, :F], wg, "dgate", tol=3e-2); check_close(dgu[:, F:], wu, "dup", tol=3e-2)


@pytest.mark.parametrize("T,S,H,KH,d", [(4096, 1024, 8, 8, 256), (8192, 4096, 6, 2, 192), (512, 256, 2, 2, 128), (8192, 2048, 5, 3, 128)])
def test_qkv_projection_with_rope_in_the_epilogue(T, S, H, KH, d):
    """The q|k|v GEMM with RoPE in its epilogue must equal GEMM + qk_rope_fwd (in place on the q and
    k heads) bit for bit: same projection tile, same fp32 rotation of the bf16-rounded values; v is
    untouched.  Cases: fused shapes (>= 128 tiles, even head count), a small one and an odd head
    count that take the unfused path, and the oracle on one of them."""
    ops = _ops()
    say(f"qkv+rope T{T} S{S} H{H} K{KH} d{d}")
    N = (H + 2 * KH) * 128
    x = bfr(T, d, seed=1).cuda(); w = bfr(N, d, seed=2, scale=d ** -0.5).cuda()
    cos, sin = ops.rope_tables(S, 128, 10000.0, "cuda")
    plain = ops.gemm(x, w)
    want = plain.clone()
    ops.qk_rope_fwd(want[:, :(H + KH) * 128], cos, sin, heads=H + KH, head_dim=128, seq_len=S, out=want[:, :(H + KH) * 128])
    got = ops.qkv_rope_proj(x, w, cos, sin, rope_heads=H + KH, seq_len=S)
    assert torch.equal(got[:, (H + KH) * 128:], plain[:, (H + KH) * 128:])
    assert torch.equal(got, want)
    if T <= 512:
        q = ref.linear_fwd(x.cpu().double(), w.cpu().double(), rt)[:, :(H + KH) * 128].reshape(T // S, S, H + KH, 128)
        rq = ref.rope_fwd(q, cos.cpu(), sin.cpu(), rt)
        assert maxrel(got[:, :(H + KH) * 128], rq.reshape(T, -1)) < 2e-2


ATTN_CASES = [
    # B, S, H, KH, D, window, softcap
    (2, 256, 4, 4, 128, None, 0.0),
    (1, 384, 4, 2, 128, None, 0.0),
    (1, 320, 4, 2, 128, 100, 0.0),
    (1, 256, 2, 1, 128, 64, 30.0),
    (1, 200, 2, 2, 128, None, 0.0),     # ragged: not a multiple of the tile
    (1, 130, 2, 1, 128, 7, 0.0),
    (2, 48, 4, 4, 64, None, 0.0),       # generic head_dim path
    (1, 40, 4, 2, 16, 9, 5.0),
]


# The lengths the benchmark configurations run at: 64 key tiles per query tile, so the far-tile
# skipping (window start, per-wave visibility), the lazy rescale over many tiles and the 1024-token
# window of the local layers all bind.  The brute-force float64 oracle needs a few seconds each.
ATTN_LONG_CASES = [
    (1, 4096, 2, 1, 128, 1024, 0.0),
    (1, 4096, 2, 1, 128, None, 50.0),
    (1, 4096, 2, 2, 128, None, 0.0),
    (1, 4000, 2, 1, 128, 1024, 0.0),    # ragged: last tiles partly outside the sequence
    (1, 4096, 2, 1, 128, 4096, 50.0),   # window as long as the sequence: equals global causal
]


@pytest.mark.parametrize("B,S,H,KH,D,window,softcap", ATTN_CASES + ATTN_LONG_CASES)
def test_attention_fwd_bwd(B, S, H, KH, D, window, softcap):
    ops = _ops()
    say(f"attn B{B} S{S} H{H} KH{KH} D{D} w{window} cap{softcap}")
    q = bfr(B * S, H * D, seed=1); k = bfr(B * S, KH * D, seed=2); v = bfr(B * S, KH * D, seed=3)
    do = bfr(B * S, H * D, seed=4)
    o, lse = ops.attn_fwd(q.cuda(), k.cuda(), v.cuda(), B=B, S=S, H=H, KH=KH, D=D, window=window, softcap=softcap)
    q4, k4, v4 = q.double().reshape(B, S, H, D), k.double().reshape(B, S, KH, D), v.double().reshape(B, S, KH, D)
    wo, wlse = ref.attention_fwd(q4, k4, v4, window=window, softcap=softcap)
    assert maxrel(o, wo.reshape(B * S, H * D)) < 1e-2, "o"
    assert (lse.cpu().double() - wlse).abs().max() < 2e-3, "lse"
    # first query attends to key 0 only
    assert maxrel(o.reshape(B, S, H, D)[:, 0], v4.repeat_interleave(H // KH, 2)[:, 0]) < 1e-2
    dq, dk, dv = ops.attn_bwd(q.cuda(), k.cuda(), v.cuda(), o, lse, do.cuda(), B=B, S=S, H=H, KH=KH, D=D,
                              window=window, softcap=softcap)
    wdq, wdk, wdv = ref.attention_bwd(q4, k4, v4, wo, wlse, do.double().reshape(B, S, H, D), window=window, softcap=softcap)
    check_close(dq, wdq.reshape(B * S, H * D), "dq", tol=2e-2, cos=0.999)
    check_close(dk, wdk.reshape(B * S, KH * D), "dk", tol=2e-2, cos=0.999)
    check_close(dv, wdv.reshape(B * S, KH * D), "dv", tol=2e-2, cos=0.999)


def test_attention_on_strided_qkv_views():
    ops = _ops()
    say("attn on fused-qkv column views")
    B, S, H, KH, D = 1, 256, 4, 2, 128
    qkv = bfr(B * S, (H + 2 * KH) * D, seed=9).cuda()
    q, k, v = qkv[:, : H * D], qkv[:, H * D:(H + KH) * D], qkv[:, (H + KH) * D:]
    o, lse = ops.attn_fwd(q, k, v, B=B, S=S, H=H, KH=KH, D=D)
    o2, lse2 = ops.attn_fwd(q.contiguous(), k.contiguous(), v.contiguous(), B=B, S=S, H=H, KH=KH, D=D)
    assert torch.equal(o, o2) and torch.equal(lse, lse2)


def test_attention_bwd_on_unaligned_views_stays_inside_its_workspace():
    """head_dim 128 on views that are not 16-byte aligned takes the generic kernels, whose fp32
    dK/dV accumulators live in the workspace behind delta: the size query must cover them, the
    results must match the aligned call, and a workspace that only holds delta is refused on
    the host (no launch)."""
    import ctypes
    ops = _ops()
    from olmax_amd import _lib
    from olmax_amd._lib import OlmaxHipError, i32, i64, f32, ptr, stream_ptr
    say("attn bwd on unaligned D=128 views")
    B, S, H, KH, D = 1, 64, 2, 1, 128
    wide = lambda cols, seed: bfr(B * S, cols + 8, seed=seed).cuda()
    bq, bk, bv, bdo = wide(H * D, 1), wide(KH * D, 2), wide(KH * D, 3), wide(H * D, 4)
    q, k, v, do = bq[:, 4:4 + H * D], bk[:, 4:4 + KH * D], bv[:, 4:4 + KH * D], bdo[:, 4:4 + H * D]
    assert q.data_ptr() % 16 == 8
    o, lse = ops.attn_fwd(q, k, v, B=B, S=S, H=H, KH=KH, D=D)
    qa, ka, va, doa = q.contiguous(), k.contiguous(), v.contiguous(), do.contiguous()
    oa, lsea = ops.attn_fwd(qa, ka, va, B=B, S=S, H=H, KH=KH, D=D)
    assert maxrel(o, oa) < 1e-2 and (lse - lsea).abs().max().item() < 2e-3
    guard = torch.full((1 << 20,), 7, dtype=torch.uint8, device="cuda")  # allocated right behind the call's buffers
    dq, dk, dv = ops.attn_bwd(q, k, v, o, lse, do, B=B, S=S, H=H, KH=KH, D=D)
    dqa, dka, dva = ops.attn_bwd(qa, ka, va, oa, lsea, doa, B=B, S=S, H=H, KH=KH, D=D)
    check_close(dq, dqa, "dq", tol=2e-2, cos=0.999); check_close(dk, dka, "dk", tol=2e-2, cos=0.999)
    check_close(dv, dva, "dv", tol=2e-2, cos=0.999)
    assert bool((guard == 7).all())
    L = _lib.load()
    L.olmax_attn_bwd_workspace_bytes.restype = ctypes.c_int64
    full = L.olmax_attn_bwd_workspace_bytes(i32(B), i32(S), i32(H), i32(KH), i32(D))
    delta_only = (B * H * S * 4 + 255) // 256 * 256
    assert full >= delta_only + 2 * B * S * KH * D * 4
    ws = torch.empty(delta_only, dtype=torch.uint8, device="cuda")
    def call(qq, kk, vv, oo, dd, nbytes):
        return L.olmax_attn_bwd(stream_ptr(), ptr(qq), ptr(kk), ptr(vv), ptr(oo), ptr(lse), ptr(dd), ptr(dq), ptr(dk), ptr(dv),
                                ptr(ws), i64(nbytes), i32(B), i32(S), i32(H), i32(KH), i32(D), i64(qq.stride(0)), i64(kk.stride(0)),
                                i64(vv.stride(0)), i64(oo.stride(0)), i64(dd.stride(0)), i64(dq.stride(0)), i64(dk.stride(0)),
                                i64(dv.stride(0)), i32(-1), f32(0.0))
    assert call(q, k, v, o, do, delta_only) == -5 and b"generic path" in L.olmax_last_error_string()
    assert call(qa, ka, va, oa, doa, delta_only) == 0  # aligned operands: the MFMA path needs delta only
    torch.cuda.synchronize()


@pytest.mark.parametrize("T,V,f32", [(33, 4096, False), (17, 1000, True), (8, 50, False), (5, 100352, False), (3, 128256, False),
                                     (3, 262144, False), (6, 1003, False), (4, 4104, True)])
@pytest.mark.parametrize("cap", [0.0, 30.0])
def test_cross_entropy(T, V, f32, cap):
    ops = _ops()
    say(f"ce T{T} V{V} f32{f32} cap{cap}")
    g = torch.Generator().manual_seed(1)
    logits = (torch.randn(T, V, generator=g) * 3)
    logits = logits if f32 else logits.to(BF)
    labels = torch.randint(0, V, (T,), generator=g, dtype=torch.int32)
    labels[1] = -100
    labels[2] = V  # out of range: zero loss, zero grad, counted
    loss, d, lse = ops.cross_entropy(logits.cuda(), labels.cuda(), softcap=cap)
    wl, wlse, n = ref.cross_entropy_fwd(logits.double(), labels.long(), softcap=cap)
    assert abs(loss.item() - wl.item()) < 2e-3 * max(1.0, abs(wl.item()))
    wd = ref.cross_entropy_bwd(logits.double(), labels.long(), softcap=cap)
    check_close(d, wd, "dlogits", tol=1e-2 if not f32 else 1e-4)
    assert d[1].abs().max().item() == 0 and d[2].abs().max().item() == 0
    mask = (labels != -100).double()
    assert ((lse.cpu().double() - wlse * mask).abs().max()) < 2e-3


@pytest.mark.parametrize("V,f32", [(100352, False), (4096, False), (262144, False), (4104, True)])
def test_cross_entropy_in_place_equals_out_of_place(V, f32):
    """dlogits may alias logits (olmax_lmhead_ce always calls it that way).  The label's logit is
    taken before any wave can store a gradient over the row, so the aliased call must give
    bit-identical loss, lse and gradient; labels sit in the first and the last 128-bit vector of
    the row, where a late re-read of the row would meet the earliest and the latest stores.
    Covers the register-resident kernels (8 and 16 waves per row) and the streaming one."""
    ops = _ops()
    say(f"ce in place == out of place V{V} f32{f32}")
    T = 64
    g = torch.Generator().manual_seed(7)
    logits = (torch.randn(T, V, generator=g) * 3)
    logits = (logits if f32 else logits.to(BF)).cuda()
    labels = torch.randint(0, V, (T,), generator=g, dtype=torch.int32)
    labels[0::4] = torch.randint(0, 8, (T // 4,), generator=g, dtype=torch.int32)          # first vector
    labels[1::4] = V - 1 - torch.randint(0, 8, (T // 4,), generator=g, dtype=torch.int32)  # last vector
    labels = labels.cuda()
    for cap in (0.0, 30.0):
        l0, d0, lse0 = ops.cross_entropy(logits, labels, softcap=cap)
        z = logits.clone()
        l1, d1, lse1 = ops.cross_entropy(z, labels, softcap=cap, inplace=True)
        assert d1.data_ptr() == z.data_ptr()
        assert l0.item() == l1.item() and torch.equal(lse0, lse1) and torch.equal(d0, d1)
        # and the loss is the mean of lse - z[label] over the rows
        zl = logits.float().gather(1, labels.long()[:, None])[:, 0]
        if cap:
            zl = cap * torch.tanh(zl / cap)
        assert abs(l0.item() - (lse0 - zl).mean().item()) < 1e-4


@pytest.mark.parametrize("T,V,f32", [(33, 4096, False), (7, 100352, False), (5, 1003, False), (9, 4104, True), (3, 262144, False)])
def test_cross_entropy_sum_and_none_reductions(T, V, f32):
    """reduction "sum" and "none" of cross_entropy_loss (src/olmax/nn/functional.py:84-91), forward and
    backward (scalar cotangent, and per-row cotangents for "none"), against the oracle."""
    ops = _ops()
    say(f"ce reductions T{T} V{V} f32{f32}")
    g = torch.Generator().manual_seed(2)
    logits = torch.randn(T, V, generator=g) * 3
    logits = logits if f32 else logits.to(BF)
    labels = torch.randint(0, V, (T,), generator=g, dtype=torch.int32)
    labels[1] = -100
    labels[2] = V
    tol = 1e-4 if f32 else 1e-2
    loss, d, _ = ops.cross_entropy(logits.cuda(), labels.cuda(), reduction="sum", dloss=0.5)
    wl = ref.cross_entropy_fwd(logits.double(), labels.long(), reduction="sum")[0]
    assert abs(loss.item() - wl.item()) < 2e-3 * max(1.0, abs(wl.item()))
    check_close(d, ref.cross_entropy_bwd(logits.double(), labels.long(), dloss=0.5, reduction="sum"), "dlogits sum", tol=tol)
    w = torch.randn(T, generator=g)
    loss, d, _ = ops.cross_entropy(logits.cuda(), labels.cuda(), reduction="none", dloss_rows=w.cuda())
    wl = ref.cross_entropy_fwd(logits.double(), labels.long(), reduction="none")[0]
    assert loss.shape == (T,) and (loss.cpu().double() - wl).abs().max() < 2e-3
    assert loss[1].item() == 0 and loss[2].item() == 0
    check_close(d, ref.cross_entropy_bwd(logits.double(), labels.long(), dloss=w.double(), reduction="none"), "dlogits none", tol=tol)
    # mean == sum / counted rows
    lm, _, _ = ops.cross_entropy(logits.cuda(), labels.cuda(), want_grad=False)
    ls, _, _ = ops.cross_entropy(logits.cuda(), labels.cuda(), want_grad=False, reduction="sum")
    assert abs(lm.item() * (T - 1) - ls.item()) < 1e-4 * abs(ls.item())


def test_cross_entropy_reference_invariants():
    """src/test/nn/functional_test.py:10-18: an appended ignore_index row leaves the mean unchanged."""
    ops = _ops()
    say("ce invariants")
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(6, 64, generator=g)
    labels = torch.randint(0, 64, (6,), generator=g, dtype=torch.int32)
    l1, _, _ = ops.cross_entropy(logits.cuda(), labels.cuda(), want_grad=False)
    l2, _, lse = ops.cross_entropy(torch.cat([logits, torch.randn(1, 64, generator=g)]).cuda(),
                                   torch.cat([labels, torch.tensor([-100], dtype=torch.int32)]).cuda(), want_grad=False)
    assert abs(l1.item() - l2.item()) < 1e-6
    lu, _, _ = ops.cross_entropy(torch.zeros(4, 64).cuda(), torch.tensor([0, 1, 2, 3], dtype=torch.int32).cuda(), want_grad=False)
    assert abs(lu.item() - math.log(64)) < 1e-5


@pytest.mark.parametrize("T,d,V,cap", [(256, 128, 1024, 0.0), (128, 256, 512, 30.0), (40, 24, 100, 0.0)])
def test_lmhead_ce(T, d, V, cap):
    ops = _ops()
    say(f"lmhead_ce T{T} d{d} V{V} cap{cap}")
    h = bfr(T, d, seed=1); W = bfr(V, d, seed=2, scale=0.1)
    labels = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(3), dtype=torch.int32)
    labels[0] = -100
    loss, dh, dW = ops.lmhead_ce(h.cuda(), W.cuda(), labels.cuda(), softcap=cap)
    wl, wdh, wdw = ref.lm_head_ce(h.double(), W.double(), labels.long(), softcap=cap, rt=rt)
    assert abs(loss.item() - wl.item()) < 1e-2 * abs(wl.item())
    check_close(dh, wdh, "dh", tol=2e-2, cos=0.999); check_close(dW, wdw, "dW", tol=2e-2, cos=0.999)


def test_embedding():
    ops = _ops()
    say("embedding gather / scatter-add")
    V, d = 50, 64
    W = bfr(V, d, seed=1)
    ids = torch.tensor([3, 7, 3, 49, 0, 3], dtype=torch.int32)
    out = ops.embed_fwd(ids.cuda(), W.cuda())
    assert torch.equal(out.cpu(), W[ids.long()])  # index work is bit-exact
    dh = bfr(6, d, seed=2)
    dW = ops.embed_bwd(ids.cuda(), dh.cuda(), V)
    want = ref.embed_bwd(ids, dh.double(), V)
    assert (dW.cpu().double() - want).abs().max() < 1e-5
    # ids outside [0, V): NumPy/JAX indexing (negative counts from the end, the rest is clamped),
    # and the scatter-add is the transpose of that gather
    odd = torch.tensor([-1, V, V + 5, -V - 3, 2], dtype=torch.int32)
    rows = torch.tensor([V - 1, V - 1, V - 1, 0, 2])
    assert torch.equal(ops.embed_fwd(odd.cuda(), W.cuda()).cpu(), W[rows])
    dh5 = bfr(5, d, seed=4)
    assert (ops.embed_bwd(odd.cuda(), dh5.cuda(), V).cpu().double() - ref.embed_bwd(rows, dh5.double(), V)).abs().max() < 1e-5
    # odd width goes through the scalar path
    W2 = bfr(V, 13, seed=3)
    assert torch.equal(ops.embed_fwd(ids.cuda(), W2.cuda()).cpu(), W2[ids.long()])


@pytest.mark.parametrize("n,gbf", [(4096, True), (1003, False), (7, True)])
def test_adamw(n, gbf):
    ops = _ops()
    say(f"adamw n{n} gbf16{gbf}")
    gen = torch.Generator().manual_seed(1)
    p = torch.randn(n, generator=gen); m = torch.zeros(n); v = torch.zeros(n)
    pc, mc, vc = p.cuda(), m.cuda(), v.cuda()
    sh = torch.empty(n, dtype=BF).cuda()
    pd, md, vd = p.double(), m.double(), v.double()
    for step in range(1, 4):
        g = torch.randn(n, generator=gen) * 0.1
        g = g.to(BF) if gbf else g
        ops.adamw_(pc, g.cuda(), mc, vc, step=step, lr=3e-3, b1=0.9, b2=0.95, eps=1e-8, wd=0.1, shadow=sh)
        pd, md, vd = ref.adamw_step(pd, g.double(), md, vd, step=step, lr=3e-3, b1=0.9, b2=0.95, eps=1e-8, wd=0.1)
    assert (pc.cpu().double() - pd).abs().max() < 1e-5
    assert (mc.cpu().double() - md).abs().max() < 1e-6 and (vc.cpu().double() - vd).abs().max() < 1e-7
    assert torch.equal(sh.cpu(), pc.cpu().to(BF))
    # g = 0 -> pure decoupled decay; wd = 0 and |g| >> eps at step 1 -> -lr * sign(g)
    p0 = torch.full((8,), 2.0).cuda(); z = torch.zeros(8).cuda()
    ops.adamw_(p0, torch.zeros(8).cuda(), z.clone(), z.clone(), step=1, lr=0.1, wd=0.5)
    assert (p0.cpu() - 2.0 * 0.95).abs().max() < 1e-6
    p1 = torch.zeros(8).cuda()
    ops.adamw_(p1, torch.tensor([1., -2., 3., -4., 5., -6., 7., -8.]).cuda(), z.clone(), z.clone(), step=1, lr=0.1, wd=0.0)
    assert (p1.cpu() - torch.tensor([-0.1, 0.1] * 4)).abs().max() < 1e-6


def test_adamw_with_device_resident_hyperparameters():
    """olmax_adamw_dev reads lr and the two bias corrections from device memory (hosts whose schedule
    and step count are device values): with the same three floats it must equal olmax_adamw bit for bit."""
    ops = _ops()
    from olmax_amd import _lib
    from olmax_amd._lib import f32, i32, i64, ptr, stream_ptr, check
    say("adamw hyper_dev")
    n, step, lr, b1, b2 = 5003, 7, 3e-3, 0.9, 0.95
    gen = torch.Generator().manual_seed(1)
    p = torch.randn(n, generator=gen); m = torch.randn(n, generator=gen) * 0.01; v = torch.rand(n, generator=gen) * 1e-4
    g = (torch.randn(n, generator=gen) * 0.1).to(BF)
    a = [t.clone().cuda() for t in (p, m, v)]
    b = [t.clone().cuda() for t in (p, m, v)]
    sa, sb = torch.empty(n, dtype=BF).cuda(), torch.empty(n, dtype=BF).cuda()
    ops.adamw_(a[0], g.cuda(), a[1], a[2], step=step, lr=lr, b1=b1, b2=b2, eps=1e-8, wd=0.1, shadow=sa)
    # the host path forms 1 - b^t in double from the fp32 values of b1 / b2 and rounds once
    f = lambda x: float(torch.tensor(x, dtype=torch.float32))
    hyper = torch.tensor([lr, 1.0 - f(b1) ** step, 1.0 - f(b2) ** step], dtype=torch.float64).to(torch.float32).cuda()
    check(_lib.load().olmax_adamw_dev(stream_ptr(), ptr(b[0]), ptr(g.cuda()), ptr(b[1]), ptr(b[2]), ptr(sb), i64(n), i32(1),
                                      f32(b1), f32(b2), f32(1e-8), f32(0.1), ptr(hyper), ptr(None)))
    torch.cuda.synchronize()
    for x, y in zip(a + [sa], b + [sb]):
        assert torch.equal(x, y)


def test_two_host_threads_on_their_own_streams_get_single_thread_results():
    """The entry points are re-entrant: they enqueue on the stream they are given, keep no
    per-call state outside their arguments and report errors through a thread-local string.
    Two host threads (ctypes releases the GIL during a call) each drive GEMM, RMSNorm and the
    attention forward / backward on a stream of their own, 25 rounds; every result must be
    bit-identical to the one the same inputs give from a single thread (these kernels use no
    atomics), and an argument error raised in one thread must not show up in the other."""
    import threading
    ops = _ops()
    from olmax_amd import _lib
    say("two host threads, two streams")
    B, S, H, KH, D = 1, 512, 2, 1, 128

    def inputs(seed):
        return dict(a=bfr(512, 256, seed=seed).cuda(), b=bfr(768, 256, seed=seed + 1).cuda(),
                    x=bfr(300, 4096, seed=seed + 2).cuda(), w=bfr(4096, seed=seed + 3).cuda(),
                    q=bfr(B * S, H * D, seed=seed + 4).cuda(), k=bfr(B * S, KH * D, seed=seed + 5).cuda(),
                    v=bfr(B * S, KH * D, seed=seed + 6).cuda(), do=bfr(B * S, H * D, seed=seed + 7).cuda())

    def work(t):
        c = ops.gemm(t["a"], t["b"])
        y = ops.rms_norm_fwd(t["x"], t["w"], 1e-6)
        o, lse = ops.attn_fwd(t["q"], t["k"], t["v"], B=B, S=S, H=H, KH=KH, D=D)
        dq, dk, dv = ops.attn_bwd(t["q"], t["k"], t["v"], o, lse, t["do"], B=B, S=S, H=H, KH=KH, D=D)
        return [c, y, o, lse, dq, dk, dv]

    ins = [inputs(10), inputs(20)]
    want = [work(t) for t in ins]
    torch.cuda.synchronize()
    errors, seen = [], [None, None]

    def run(idx):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for it in range(25):
                    got = work(ins[idx])
                    if idx == 0 and it == 5:  # an argument error in this thread only
                        try:
                            ops.attn_fwd(ins[0]["q"], ins[0]["k"], ins[0]["v"], B=B, S=S, H=3, KH=2, D=D)
                        except _lib.OlmaxHipError as e:
                            seen[0] = str(e)
                    stream.synchronize()
                    for g, w_ in zip(got, want[idx]):
                        if not torch.equal(g, w_):
                            errors.append((idx, it))
                if idx == 1:
                    seen[1] = _lib.load().olmax_last_error_string().decode()
        except Exception as e:  # noqa: BLE001 - reported below, in the main thread
            errors.append((idx, repr(e)))

    threads = [threading.Thread(target=run, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads)
    assert not errors, errors
    assert seen[0], "the bad call in thread 0 must raise"
    assert seen[1] == "", f"thread 1 saw another thread's error: {seen[1]!r}"
