"""The hybrid-mixer HIP kernels (jax_llama_amd._C_hybrid) against the PyTorch implementation of the same ops
(ops/hybrid.py CPU path), at sizes that are not multiples of the tile shapes, in both number formats."""
import pytest
import torch

from jax_llama_amd.ops import hybrid as hy

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def _tol(dt):
    return 2e-5  # both paths round the operands alike: only the summation order differs


def _close(a, b, tol, what=""):
    a, b = a.float().cpu(), b.float().cpu()
    assert a.shape == b.shape, f"{what}: shapes {tuple(a.shape)} vs {tuple(b.shape)}"
    if a.numel() == 0:
        return
    err = float((a - b).abs().max() / b.abs().max().clamp_min(1e-6))
    assert err <= tol, f"{what}: relative error {err:.3e} > {tol:.1e}"


def _rand(*shape, dt=torch.float32, std=1.0):
    return (torch.randn(*shape) * std).to(dt)


def test_extension_loaded():
    assert hy.ext_available() and hy.so_path().endswith(".so")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m,n,k", [(1, 7, 24), (3, 64, 320), (8, 130, 72), (9, 4, 320), (70, 392, 320), (200, 96, 24),
                                   (129, 64, 257), (600, 200, 96), (513, 130, 320)])
def test_linear(dt, m, n, k):
    x, w = _rand(m, k), _rand(n, k, dt=dt, std=k ** -0.5)
    _close(hy.linear(x.to(DEV), w.to(DEV)), hy.linear(x, w), _tol(dt), "linear")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m", [2, 8, 77, 530])
def test_linear_swiglu_strided_rows(dt, m):
    k, n = 96, 40
    big = _rand(m, k + 32)
    w = _rand(2 * n, k, dt=dt, std=k ** -0.5)
    got = hy.linear(big.to(DEV)[:, 16:16 + k], w.to(DEV), swiglu=True)
    _close(got, hy.linear(big[:, 16:16 + k], w, swiglu=True), _tol(dt), "swiglu")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m,top,e", [(1, 2, 8), (4, 2, 8), (3, 1, 1), (150, 2, 8), (90, 3, 5), (300, 1, 4),
                                     (20, 2, 8), (21, 3, 2), (9, 1, 1), (700, 2, 3)])
def test_moe_table(dt, m, top, e):
    d, ff, v = 72, 40, 50
    x = _rand(m, d)
    ids = torch.randint(0, v, (m,), dtype=torch.int32)
    table = torch.stack([torch.randperm(e)[:top] for _ in range(v)]).to(torch.int32)
    w_gu, w_down = _rand(e, 2 * ff, d, dt=dt, std=d ** -0.5), _rand(e, d, ff, dt=dt, std=ff ** -0.5)
    got = hy.moe_table(x.to(DEV), ids.to(DEV), table.to(DEV), w_gu.to(DEV), w_down.to(DEV))
    # bf16: the hidden activation is rounded to bf16 before the down projection on both paths, but the two paths'
    # fp32 sums differ in order, so a hidden value can round to the neighbouring bf16
    _close(got, hy.moe_table(x, ids, table, w_gu, w_down), 2e-5 if dt == torch.float32 else 4e-3, "moe")


@pytest.mark.parametrize("wn", [1, 50])
@pytest.mark.parametrize("nsum", [1, 3])
def test_norm_residual(wn, nsum):
    m, d = 5, 50
    x, y, w = _rand(m, d), _rand(m * nsum, d), torch.rand(wn) + 0.5
    got = hy.norm_residual_(x.clone().to(DEV), y.to(DEV), w.to(DEV), 1e-6, nsum, 1.0 / nsum)
    _close(got, hy.norm_residual_(x.clone(), y, w, 1e-6, nsum, 1.0 / nsum), 1e-5, "norm_residual")
    _close(hy.rms_rows(y.to(DEV), w.to(DEV), 1e-6), hy.rms_rows(y, w, 1e-6), 1e-5, "rms_rows")


@pytest.mark.parametrize("dt", DTYPES)
def test_embed_and_side_gate(dt):
    v, d, m = 40, 30, 6
    table = _rand(v, 3 * d, dt=dt)
    ids = torch.randint(0, v, (m,), dtype=torch.int32)
    _close(hy.embed_rows(ids.to(DEV), table.to(DEV), d, d), hy.embed_rows(ids, table, d, d), 0.0, "embed")
    gp = _rand(m, d)
    _close(hy.gelu_gate_rows(gp.to(DEV), ids.to(DEV), table.to(DEV), 2 * d), hy.gelu_gate_rows(gp, ids, table, 2 * d),
           1e-5, "gelu gate")


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("shape", [dict(b=1, s=1, s0=0, h=4, g=2, dim=64, vdim=64),
                                   dict(b=2, s=5, s0=0, h=3, g=1, dim=24, vdim=40),
                                   dict(b=1, s=70, s0=130, h=4, g=4, dim=72, vdim=136),
                                   dict(b=2, s=1, s0=300, h=6, g=2, dim=32, vdim=16),
                                   dict(b=1, s=70, s0=130, h=4, g=2, dim=64, vdim=128),   # the MFMA prefill shapes
                                   dict(b=2, s=203, s0=0, h=2, g=1, dim=128, vdim=64),
                                   dict(b=1, s=33, s0=31, h=2, g=2, dim=128, vdim=128)])
@pytest.mark.parametrize("own_kv", [True, False])
def test_attention(dt, shape, own_kv):
    b, s, s0, h, g, dim, vdim = (shape[k] for k in ("b", "s", "s0", "h", "g", "dim", "vdim"))
    t, eps = s0 + s + 3, 1e-6
    kc, vc = _rand(b, g, t, dim, dt=dt), _rand(b, g, t, vdim, dt=dt)
    cols = h * dim + (g * (dim + vdim) if own_kv else 0)
    proj = _rand(b * s, cols)
    pos = (torch.arange(s0, s0 + s, dtype=torch.int32)[None] + torch.zeros(b, 1, dtype=torch.int32)).contiguous()
    bias = hy.distance_bias_table(_rand(10, h), 37)
    kc_g, vc_g = kc.to(DEV), vc.to(DEV)
    q_ref = hy.attn_prep(proj, pos, s0, b, s, h, g, dim, vdim, kc if own_kv else None, vc if own_kv else None, eps,
                         0.3, 4)
    q_got = hy.attn_prep(proj.to(DEV), pos.to(DEV), s0, b, s, h, g, dim, vdim, kc_g if own_kv else None,
                         vc_g if own_kv else None, eps, 0.3, 4)
    _close(q_got, q_ref, 1e-5, "q")
    _close(kc_g, kc, 1e-5 if dt == torch.float32 else 8e-3, "k cache")
    _close(vc_g, vc, 1e-5 if dt == torch.float32 else 8e-3, "v cache")
    # the attention itself on identical caches
    kc_g, vc_g = kc.to(DEV), vc.to(DEV)
    # bf16 caches at the MFMA shapes: q is rounded to bf16 for the score product (the reference gets the same q)
    mma = dt == torch.bfloat16 and s > 1 and dim in (64, 128) and vdim in (64, 128)
    for cap, b_ in ((5.0, bias), (0.0, None)):
        ref = hy.attn_bias(q_ref.to(torch.bfloat16).float() if mma else q_ref, kc, vc, s0, 0.25, cap, b_)
        got = hy.attn_bias(q_ref.to(DEV), kc_g, vc_g, torch.tensor([s0], dtype=torch.int32, device=DEV), 0.25, cap,
                           b_.to(DEV) if b_ is not None else None)
        _close(got, ref, 2e-4 if mma else 2e-5, "attention")  # (MFMA path: v_exp_f32 and exp-based tanh)


@pytest.mark.parametrize("shape", [dict(b=1, s=1, h=4, g=2, dim=32, vdim=32, taps=4),
                                   dict(b=2, s=2, h=2, g=1, dim=40, vdim=24, taps=4),
                                   dict(b=1, s=37, h=6, g=3, dim=128, vdim=72, taps=3),
                                   dict(b=2, s=9, h=2, g=2, dim=16, vdim=130, taps=1)])
def test_delta_rule(shape):
    b, s, h, g, dim, vdim, taps = (shape[k] for k in ("b", "s", "h", "g", "dim", "vdim", "taps"))
    c = 2 * g * dim + h * vdim
    proj = _rand(b * s, c + h * vdim + 2 * h + 5)[:, :c + h * vdim + 2 * h]  # strided rows
    conv_w, tail = _rand(c, taps, std=0.6), _rand(b, c, max(taps - 1, 0))
    a_log, dt_bias = torch.rand(h) - 1.0, torch.randn(h)
    state = _rand(b, h, dim, vdim, std=0.3)
    tail_g, state_g = tail.clone().to(DEV), state.clone().to(DEV)
    ref = hy.delta_prep(proj, b, s, h, g, dim, vdim, conv_w, tail, a_log, dt_bias)
    got = hy.delta_prep(proj.to(DEV), b, s, h, g, dim, vdim, conv_w.to(DEV), tail_g, a_log.to(DEV), dt_bias.to(DEV))
    for r, x, name in zip(ref, got, ("q", "k", "v", "beta", "decay")):
        _close(x, r, 2e-5, name)
    _close(tail_g, tail, 0.0, "conv tail")
    o_ref = hy.delta_scan(*ref, state, b, s)
    o_got = hy.delta_scan(*(x.to(DEV) for x in ref), state_g, b, s)
    _close(o_got, o_ref, 5e-5, "delta o")
    _close(state_g, state, 5e-5, "delta state")
    gate, w = _rand(b * s, h * vdim), torch.rand(vdim) + 0.5
    _close(hy.gated_rmsnorm(o_ref.to(DEV), gate.to(DEV), w.to(DEV), 1e-6), hy.gated_rmsnorm(o_ref, gate, w, 1e-6), 2e-5,
           "gated norm")


@pytest.mark.parametrize("m,n,k", [(256, 64, 96), (777, 400, 320), (2048, 16, 32)])
def test_linear_on_the_packed_gemm(m, n, k):
    """Prompt-sized dense bf16 linears go to the framework's fragment-packed MFMA GEMM when the main extension is
    built; same operands, so the result matches the row-major kernel and the CPU op up to summation order."""
    from jax_llama_amd import ops
    x, w = _rand(m, k), _rand(n, k, dt=torch.bfloat16, std=k ** -0.5)
    xg, wg = x.to(DEV), w.to(DEV)
    assert hy._use_packed_gemm(xg, wg) == ops.ext_available()
    got = hy.linear(xg, wg)
    _close(got, hy.linear(x, w), 2e-5, "packed gemm vs cpu")
    hy.PACKED_GEMM = False
    try:
        _close(hy.linear(xg, wg), got, 2e-5, "row-major kernel vs packed gemm")
    finally:
        hy.PACKED_GEMM = True
    assert not hy._use_packed_gemm(xg[:100], wg) and not hy._use_packed_gemm(xg, wg[:15])
