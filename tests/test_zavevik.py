"""Zavevik through the framework (model, cache, stepper, engine) against the plain float64 oracle
(tests/oracle_zavevik.py), on the CPU op path and, marked gpu, on the HIP kernels. Small configurations built here:
sizes that are not multiples of any tile, unequal key / value widths, one and several lanes per recurrent column,
top-1 / top-3 routing, a layer without feed-forward, shared keys, and a model without any of the optional parts."""
import numpy as np
import pytest
import torch

import oracle_zavevik as oz
from jax_llama_amd.config import ZavevikConfig
from jax_llama_amd.models.zavevik import ZavevikForCausalLM, random_state_dict
from jax_llama_amd.ops import hybrid as hy
from jax_llama_amd.runtime.engine import GenerationConfig
from jax_llama_amd.runtime.stepper import SequenceStepper

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F32, BF16 = torch.float32, torch.bfloat16


def _moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def cfg_full():
    att = dict(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.3, softcap=6.0, bias_max=12,
               q_temp={"coef": 0.5, "every": 3})
    return {"architecture": "Zavevik", "vocab": 61, "width": 48, "norm": {"eps": 1e-6}, "token_side": {"dim": 6},
            "layers": [
                {"type": "attention", "mixer": dict(att), "mlp": _moe(5, 3, 24)},
                {"type": "delta", "mixer": dict(heads=2, kv_heads=1, dim=16, vdim=8, conv=3), "mlp": None},
                {"type": "attention", "mixer": dict(att, kv_from=0, softcap=2.5, bias_max=30, scale=0.7,
                                                    q_temp={"coef": 0.2, "every": 1}), "mlp": _moe(3, 1, 40)},
                {"type": "delta", "mixer": dict(heads=2, kv_heads=2, dim=40, vdim=8, conv=2), "mlp": _moe(5, 2, 24)},
            ]}


def cfg_bare():
    """No side input, no soft cap / bias / temperature, one head, one expert, a one-tap convolution."""
    return {"architecture": "Zavevik", "vocab": 37, "width": 40, "norm": {"eps": 1e-5},
            "layers": [
                {"type": "delta", "mixer": dict(heads=1, kv_heads=1, dim=8, vdim=72, conv=1), "mlp": _moe(1, 1, 16)},
                {"type": "attention", "mixer": dict(heads=1, kv_heads=1, dim=8, vdim=8, scale=1.0), "mlp": None},
            ]}


def build(cfg, device, dtype=F32, seed=0, buckets=8, edit=None):
    config = ZavevikConfig.from_dict(cfg)
    sd = random_state_dict(config, seed=seed, buckets=buckets)
    for k in list(sd):
        if k.endswith("mix.rel"):  # distinct, large biases: a wrong bucket or a clamp one off moves the logits
            sd[k] = (sd[k].float() * 3.0).to(BF16)
    if edit:
        edit(sd)
    model = ZavevikForCausalLM(config, device=device, dtype=dtype, _do_init=False).load_state_dict(sd)
    return model, sd


def toks(n, vocab, seed=1):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def err(got, ref):
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    d = got - ref
    return float(np.sqrt(np.mean(d * d)) / np.sqrt(np.mean(ref * ref)))


def tol(device, dtype=F32):
    return 3e-2 if dtype == BF16 else 2e-5


def run_portions(model, tokens, portions, rid="r", stepper=None, max_tokens=None):
    """Logits of every position through the stepper, the prompt cut into ``portions``."""
    st = stepper or SequenceStepper(model, max_tokens or len(tokens))
    out, at = [], 0
    for n in portions:
        out.append(st.feed(rid, tokens[at:at + n], list(range(n))).float().cpu())
        at += n
    assert at == len(tokens)
    st.end(rid)
    return torch.cat(out).numpy()


# ---------------------------------------------------------------------------------------------- mechanisms alone
def test_config_round_trip():
    c = ZavevikConfig.from_dict(cfg_full())
    assert ZavevikConfig.from_dict(c.to_dict()) == c and c.num_hidden_layers == 4
    assert c.layers[2].mixer.kv_from == 0 and c.layers[1].mlp is None and c.side_dim == 6
    bad = cfg_full()
    bad["layers"][2]["mixer"]["kv_from"] = 1  # a delta layer holds no keys
    with pytest.raises(ValueError):
        ZavevikConfig.from_dict(bad)


@pytest.mark.parametrize("nb,reach", [(8, 12), (32, 200), (6, 7), (4, 64), (16, 9)])
def test_distance_bias_table_matches_bucket_rule(nb, reach):
    rel = torch.arange(nb * 2, dtype=torch.float32).reshape(nb, 2)
    table = hy.distance_bias_table(rel, reach)
    assert table.shape == (reach + 1, 2)
    for n in range(reach + 1):
        assert table[n, 0] == rel[oz.bucket(n, nb, reach), 0], n
    assert oz.bucket(reach, nb, reach) == nb - 1 and oz.bucket(10 * reach, nb, reach) == nb - 1


@pytest.mark.parametrize("device", DEVICES)
def test_attention_mechanism(device):
    """One attention sublayer against the oracle: GQA, temperature, soft cap, far / clamped distances."""
    mc = dict(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.3, softcap=4.0, bias_max=9, q_temp={"coef": 0.7, "every": 2})
    t, d, eps = 29, 48, 1e-6
    g = torch.Generator().manual_seed(3)
    w = {"m.q": torch.randn(64, d, generator=g) * 0.4, "m.k": torch.randn(32, d, generator=g) * 0.4,
         "m.v": torch.randn(48, d, generator=g) * 0.4, "m.o": torch.randn(d, 96, generator=g) * 0.2,
         "m.rel": torch.randn(6, 4, generator=g) * 3.0}
    h = torch.randn(t, d, generator=g)
    ref = oz.attention(w, "m.", mc, h.double().numpy(), eps, oz.project_kv(w, "m.", mc, h.double().numpy(), eps))
    kc, vc = torch.zeros(1, 2, t, 16, device=device), torch.zeros(1, 2, t, 24, device=device)
    w_in = torch.cat([w["m.q"], w["m.k"], w["m.v"]]).to(device)
    bias = hy.distance_bias_table(w["m.rel"], 9).to(device)
    pos = torch.arange(t, dtype=torch.int32, device=device)
    # in two portions, the second starting inside the clamped distances
    outs = []
    for s0, s in ((0, 11), (11, 18)):
        proj = hy.linear(h[s0:s0 + s].to(device), w_in)
        q = hy.attn_prep(proj, pos[s0:s0 + s], s0, 1, s, 4, 2, 16, 24, kc, vc, eps, 0.7, 2)
        outs.append(hy.linear(hy.attn_bias(q, kc, vc, s0, 0.3, 4.0, bias), w["m.o"].to(device)).cpu())
    assert err(torch.cat(outs).numpy(), ref) < 2e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dim,vdim,heads,kv_heads,taps", [(16, 8, 2, 1, 3), (40, 24, 4, 4, 4), (8, 72, 1, 1, 1)])
def test_delta_mechanism(device, dim, vdim, heads, kv_heads, taps):
    mc = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim)
    t, d, eps = 23, 40, 1e-6
    g = torch.Generator().manual_seed(4)
    r = lambda *s, sc=0.3: torch.randn(*s, generator=g) * sc  # noqa: E731
    w = {"m.q": r(kv_heads * dim, d), "m.k": r(kv_heads * dim, d), "m.v": r(heads * vdim, d), "m.g": r(heads * vdim, d),
         "m.b": r(heads, d), "m.a": r(heads, d), "m.o": r(d, heads * vdim),
         "m.q.conv": r(kv_heads * dim, taps, sc=0.7), "m.k.conv": r(kv_heads * dim, taps, sc=0.7),
         "m.v.conv": r(heads * vdim, taps, sc=0.7), "m.A_log": r(heads, sc=1.0), "m.dt_bias": r(heads, sc=1.0),
         "m.norm": torch.rand(vdim, generator=g) + 0.5}
    h = torch.randn(t, d, generator=g)
    ref = oz.delta(w, "m.", mc, h.double().numpy(), eps)
    w_in = torch.cat([w["m." + n] for n in ("q", "k", "v", "g", "b", "a")]).to(device)
    conv = torch.cat([w[f"m.{n}.conv"] for n in ("q", "k", "v")]).to(device)
    c = 2 * kv_heads * dim + heads * vdim
    state = torch.zeros(1, heads, dim, vdim, device=device)
    tail = torch.zeros(1, c, taps - 1, device=device)
    outs = []
    for s0, s in ((0, 1), (1, 2), (3, 13), (16, 1), (17, 6)):  # portions shorter and longer than the taps
        proj = hy.linear(h[s0:s0 + s].to(device), w_in)
        q, k, v, beta, decay = hy.delta_prep(proj, 1, s, heads, kv_heads, dim, vdim, conv, tail,
                                             w["m.A_log"].to(device), w["m.dt_bias"].to(device))
        o = hy.delta_scan(q, k, v, beta, decay, state, 1, s)
        y = hy.gated_rmsnorm(o, proj[:, c:c + heads * vdim], w["m.norm"].to(device), eps)
        outs.append(hy.linear(y, w["m.o"].to(device)).cpu())
    assert err(torch.cat(outs).numpy(), ref) < 2e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("m,experts,top", [(3, 4, 2), (40, 5, 3), (70, 1, 1)])
def test_moe_and_side_mechanisms(device, m, experts, top):
    d, ff, v, sd_ = 40, 24, 19, 6
    g = torch.Generator().manual_seed(5)
    w = {"f.table": torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(v)]).to(torch.int32)}
    for e in range(experts):
        w[f"f.e{e}.gate"], w[f"f.e{e}.up"] = torch.randn(ff, d, generator=g) * 0.3, torch.randn(ff, d, generator=g) * 0.3
        w[f"f.e{e}.down"] = torch.randn(d, ff, generator=g) * 0.3
    w.update({"side.embed": torch.randn(v, 3 * sd_, generator=g), "s.gate": torch.randn(sd_, d, generator=g) * 0.3,
              "s.proj": torch.randn(d, sd_, generator=g), "s.norm": torch.rand(d, generator=g)})
    x = torch.randn(m, d, generator=g)
    ids = toks(m, v)
    fc = {"router": {"experts": experts, "top": top}}
    ref = oz.moe(w, "f.", fc, x.double().numpy(), ids)
    idt = torch.tensor(ids, dtype=torch.int32, device=device)
    w_gu = torch.stack([torch.cat([w[f"f.e{e}.gate"], w[f"f.e{e}.up"]]) for e in range(experts)]).to(device)
    w_dn = torch.stack([w[f"f.e{e}.down"] for e in range(experts)]).to(device)
    y = hy.moe_table(x.to(device), idt, w["f.table"].to(device), w_gu, w_dn)
    assert err(y.reshape(m, top, d).mean(1).cpu().numpy(), ref) < 2e-5
    ref_s = oz.side_input(w, "s.", 1, sd_, x.double().numpy(), ids, 1e-6)
    gg = hy.gelu_gate_rows(hy.linear(x.to(device), w["s.gate"].to(device)), idt, w["side.embed"].to(device), sd_)
    xs = torch.zeros(m, d, device=device)
    hy.norm_residual_(xs, hy.linear(gg, w["s.proj"].to(device)), w["s.norm"].to(device), 1e-6)
    assert err(xs.cpu().numpy(), ref_s) < 2e-5


# ---------------------------------------------------------------------------------------------- whole model
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cfg", [cfg_full, cfg_bare])
def test_prompt_logits_and_residual_stream(device, cfg):
    model, sd = build(cfg(), device)
    t = toks(45, model.config.vocab_size)
    ref, ref_hidden = oz.forward(cfg(), sd, t)
    ids = torch.tensor([t], dtype=torch.int32)
    out = model(ids, output_hidden_states=True)
    assert err(out.logits[0].cpu().numpy(), ref) < tol(device)
    for i, hs in enumerate(out.hidden_states):
        assert err(hs[0].cpu().numpy(), ref_hidden[i]) < tol(device), f"layer {i}"
    assert err(out.logits[0, :3].cpu().numpy(), ref[:3]) < tol(device)  # the first tokens of a sequence


@pytest.mark.parametrize("device", DEVICES)
def test_bfloat16_serving_format(device):
    model, sd = build(cfg_full(), device, dtype=BF16)
    t = toks(40, 61)
    ref, _ = oz.forward(cfg_full(), sd, t)
    got = run_portions(model, t, [33] + [1] * 7)
    assert err(got, ref) < tol(device, BF16)
    k, _ = model.init_cache(1, 8).layer(0)
    assert k.dtype == BF16 and model.init_cache(1, 8).recurrent(1)[0].dtype == F32


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cfg", [cfg_full, cfg_bare])
def test_prefill_against_token_by_token(device, cfg):
    model, sd = build(cfg(), device)
    t = toks(34, model.config.vocab_size, seed=2)
    ref, _ = oz.forward(cfg(), sd, t)
    whole = run_portions(model, t, [34])
    single = run_portions(model, t, [1] * 34)
    assert err(whole, ref) < tol(device) and err(single, ref) < tol(device)
    assert err(single, whole) < tol(device)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("portions", [[2] * 20, [3, 2, 9, 1, 1, 17, 2, 5], [12, 13, 14, 1], [1, 39], [38, 2]])
def test_portions_of_any_size(device, portions):
    model, sd = build(cfg_full(), device, seed=1)
    t = toks(sum(portions), 61, seed=3)
    ref, _ = oz.forward(cfg_full(), sd, t)
    assert err(run_portions(model, t, portions), ref) < tol(device)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_past_every_edge(device):
    """70 single-token steps after a short prompt: past the clamp of both distance tables, many temperature steps."""
    model, sd = build(cfg_full(), device, seed=2)
    t = toks(76, 61, seed=4)
    ref, _ = oz.forward(cfg_full(), sd, t)
    got = run_portions(model, t, [6] + [1] * 70)
    e = [err(got[i], ref[i]) for i in range(76)]
    assert max(e) < tol(device), int(np.argmax(e))


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_decides(device):
    """A large bias on the clamped (farthest) bucket of one head makes the far keys carry the softmax, in the prompt
    and while decoding; keys one inside / outside the clamp get different buckets."""
    def edit(sd):
        rel = sd["l0.mix.rel"].float()
        rel[-1, 0], rel[-2, 0] = 7.0, -7.0
        sd["l0.mix.rel"] = rel.to(BF16)
    model, sd = build(cfg_full(), device, edit=edit)
    t = toks(30, 61, seed=5)
    ref, _ = oz.forward(cfg_full(), sd, t)
    got = run_portions(model, t, [10, 3, 1, 1, 1, 14])
    assert err(got, ref) < tol(device)
    plain, _ = oz.forward(cfg_full(), build(cfg_full(), "cpu")[1], t)
    assert err(plain[13:], ref[13:]) > 1e-2  # the edit matters once distances reach the clamp


@pytest.mark.parametrize("device", DEVICES)
def test_rows_are_reset_and_reused(device):
    """A finished request's row (keys, recurrent state, convolution tail) serves the next request from a clean start;
    two live requests fed in turns do not touch each other."""
    model, sd = build(cfg_full(), device)
    a, b = toks(21, 61, seed=6), toks(17, 61, seed=7)
    ref_a, _ = oz.forward(cfg_full(), sd, a)
    ref_b, _ = oz.forward(cfg_full(), sd, b)
    st = SequenceStepper(model, 32)
    assert err(run_portions(model, a, [20, 1], "a", st), ref_a) < tol(device)
    assert st.live() == [] and len(st._free) == 1
    assert err(run_portions(model, b, [5, 12], "b", st), ref_b) < tol(device)  # the same row again
    assert len(st._free) == 1
    got_a, got_b = [], []
    for lo in range(0, 21, 3):  # interleaved: two rows live at once
        got_a.append(st.feed("a", a[lo:lo + 3], list(range(len(a[lo:lo + 3])))).cpu())
        if lo < 17:
            got_b.append(st.feed("b", b[lo:lo + 3], list(range(len(b[lo:lo + 3])))).cpu())
    assert st.live() == ["a", "b"] and st.held("a") == 21 and st.held("b") == 17
    assert err(torch.cat(got_a).numpy(), ref_a) < tol(device) and err(torch.cat(got_b).numpy(), ref_b) < tol(device)
    with pytest.raises(ValueError):
        st.feed("a", toks(12, 61), [])  # more than the row holds


@pytest.mark.parametrize("device", DEVICES)
def test_batch_rows_against_each_alone(device):
    model, sd = build(cfg_full(), device)
    rows = [toks(19, 61, seed=8), toks(19, 61, seed=9), toks(19, 61, seed=10)]
    cache = model.init_cache(3, 24)
    out = model(torch.tensor(rows, dtype=torch.int32), past_key_values=cache).logits
    nxt = [[5], [6], [7]]
    out2 = model(torch.tensor(nxt, dtype=torch.int32), past_key_values=cache).logits  # one decode step of the batch
    for r in range(3):
        ref, _ = oz.forward(cfg_full(), sd, rows[r] + nxt[r])
        assert err(out[r].cpu().numpy(), ref[:19]) < tol(device)
        assert err(out2[r].cpu().numpy(), ref[19:]) < tol(device)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cfg", [cfg_full, cfg_bare])
def test_greedy_generation_through_the_engine(device, cfg):
    """model.generate (prefill + decode steps of the engine, hipGraph replay on the GPU): every generated token is the
    oracle's argmax of the sequence so far (up to rounding between near-equal logits)."""
    model, sd = build(cfg(), device)
    v = model.config.vocab_size
    prompt = toks(9, v, seed=11)
    seq = model.generate(torch.tensor([prompt], dtype=torch.int32),
                         generation_config=GenerationConfig(max_length=30, pad_token_id=0)).sequences[0].cpu().tolist()
    assert seq[:9] == prompt and len(seq) == 30 and all(0 <= x < v for x in seq)
    ref, _ = oz.forward(cfg(), sd, seq)
    for i in range(9, 30):
        row = ref[i - 1]
        assert row.max() - row[seq[i]] <= 1e-4 * np.abs(row).max(), i
    again = model.generate(torch.tensor([prompt], dtype=torch.int32),
                           generation_config=GenerationConfig(max_length=30, pad_token_id=0)).sequences[0].cpu().tolist()
    assert again == seq  # the engine's cached cache row starts clean


def test_checkpoint_directory_round_trip(tmp_path):
    from jax_llama_amd.models import registry
    model, sd = build(cfg_full(), "cpu")
    model.save_pretrained(str(tmp_path), sd)
    assert registry.architecture_of(str(tmp_path)) == "zavevik"
    again = registry.load_model(str(tmp_path), device="cpu", dtype=F32)
    t = toks(12, 61)
    ids = torch.tensor([t], dtype=torch.int32)
    assert torch.equal(again(ids).logits, model(ids).logits)
    assert not registry.supports_dtype("llama", F32) and registry.supports_dtype("zavevik", F32)


def test_trace_runner_program(tmp_path):
    """bin/trace_run as a user starts it: steps on standard input, logits files, 'done' lines, rows given back."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    model, sd = build(cfg_full(), "cpu")
    ckpt, out = str(tmp_path / "ckpt"), str(tmp_path / "out")
    model.save_pretrained(ckpt, sd)
    a, b = toks(9, 61, seed=12), toks(5, 61, seed=13)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:6], "want": [0, 5]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[6:8], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[8:], "want": [0]}], "end": ["a"]},
             {"step": 3, "entries": [{"id": "b", "tokens": b, "want": [4]}], "end": ["b"]}]
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", ckpt, "--dtype", "float32",
                        "--out", out, "--max-tokens", "16", "--device", "cpu"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [ln for ln in p.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(4)]
    assert not os.path.exists(os.path.join(out, "1.f32"))
    ref_a, _ = oz.forward(cfg_full(), sd, a)
    ref_b, _ = oz.forward(cfg_full(), sd, b)
    got0 = np.fromfile(os.path.join(out, "0.f32"), dtype="<f4").reshape(2, 61)
    got2 = np.fromfile(os.path.join(out, "2.f32"), dtype="<f4").reshape(1, 61)
    got3 = np.fromfile(os.path.join(out, "3.f32"), dtype="<f4").reshape(1, 61)
    assert err(got0, ref_a[[0, 5]]) < 2e-5 and err(got2, ref_a[[8]]) < 2e-5 and err(got3, ref_b[[4]]) < 2e-5
    # a family without an all-fp32 path refuses that format at the start
    llama = tmp_path / "llama"
    llama.mkdir()
    (llama / "config.json").write_text(json.dumps({"model_type": "llama"}))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(llama), "--dtype",
                        "float32", "--out", out, "--device", "cpu"], input="", capture_output=True, text=True, timeout=300)
    assert r.returncode == 3


def cfg_mfma_shapes():
    """Head sizes of the MFMA attention kernels (64 / 128), three query heads per key head, six layers in another
    order, two layers on shared keys, a distance table that reaches a few hundred keys."""
    a64 = dict(heads=6, kv_heads=2, dim=64, vdim=128, scale=0.125, softcap=30.0, bias_max=300,
               q_temp={"coef": 0.3, "every": 64})
    a128 = dict(heads=2, kv_heads=1, dim=128, vdim=64, scale=0.09, bias_max=150)
    dl = dict(heads=4, kv_heads=2, dim=64, vdim=48, conv=4)
    return {"architecture": "Zavevik", "vocab": 300, "width": 192, "norm": {"eps": 1e-6}, "token_side": {"dim": 16},
            "layers": [{"type": "attention", "mixer": dict(a64), "mlp": _moe(4, 2, 96)},
                       {"type": "attention", "mixer": dict(a64, kv_from=0), "mlp": None},
                       {"type": "delta", "mixer": dict(dl), "mlp": _moe(4, 2, 96)},
                       {"type": "attention", "mixer": dict(a128), "mlp": _moe(6, 3, 64)},
                       {"type": "delta", "mixer": dict(dl, heads=2, kv_heads=1, dim=128, vdim=128), "mlp": None},
                       {"type": "attention", "mixer": dict(a128, kv_from=3, softcap=5.0), "mlp": _moe(4, 1, 96)}]}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_longer_prompts_at_the_mfma_head_sizes(dtype):
    """600 tokens in uneven portions (prompt-sized GEMMs, the flash prefill starting at unaligned slots, decode over
    several key splits) on the GPU against the framework's fp32 CPU path, which the tests above tie to the oracle."""
    cfg = cfg_mfma_shapes()
    ref_model, sd = build(cfg, "cpu", F32, buckets=32)
    t = toks(600, 300, seed=21)
    with torch.no_grad():
        ref = ref_model(torch.tensor([t], dtype=torch.int32)).logits[0].numpy()
    model = ZavevikForCausalLM(ZavevikConfig.from_dict(cfg), device="cuda", dtype=dtype, _do_init=False).load_state_dict(sd)
    portions = [261, 3, 2, 190, 64, 37] + [1] * 43
    got = run_portions(model, t, portions)
    e = [err(got[i], ref[i]) for i in range(600)]
    assert max(e) < (2e-4 if dtype == F32 else 4e-2), (int(np.argmax(e)), max(e))
    whole = run_portions(model, t, [600])
    assert err(whole, got) < (2e-5 if dtype == F32 else 2e-2)


@pytest.mark.parametrize("device", DEVICES)
def test_sampled_generation_through_the_engine(device):
    """The framework's sampler (temperature, top-k, top-p, seeded Philox) on Zavevik logits: reproducible per seed,
    different across seeds, tokens inside the vocabulary, and every token inside the top-k of the oracle's logits."""
    model, sd = build(cfg_full(), device)
    prompt = torch.tensor([toks(7, 61, seed=14)], dtype=torch.int32)
    gc = dict(max_length=27, pad_token_id=0, do_sample=True, temperature=0.9, top_k=5, top_p=0.95)
    a = model.generate(prompt, generation_config=GenerationConfig(seed=3, **gc)).sequences[0].cpu().tolist()
    b = model.generate(prompt, generation_config=GenerationConfig(seed=3, **gc)).sequences[0].cpu().tolist()
    c = model.generate(prompt, generation_config=GenerationConfig(seed=4, **gc)).sequences[0].cpu().tolist()
    assert a == b and a != c and all(0 <= x < 61 for x in a + c)
    ref, _ = oz.forward(cfg_full(), sd, a)
    for i in range(7, 27):
        row = ref[i - 1]
        assert row[a[i]] >= np.sort(row)[-5] - 1e-4 * np.abs(row).max(), i
