"""Plain, slow float64 implementation of the Zavevik decoder for the tests: one function per mechanism, written from
the equations, token loops instead of kernels, no cache (a whole sequence is recomputed from its first token) and no
code shared with the package. Inputs: the config as a plain dict (the config.json layout) and a checkpoint-named
dict of tensors.

Equations (x: residual, h: a sublayer's input = x, eps = norm.eps):
  layer        x += g1 * rms(mixer(x));  x += g2 * rms(moe(x));  x += side(x)          rms(y) = y / sqrt(mean(y^2) + eps)
  attention    q, k, v = per-head rms of W h (no gain); q *= 1 + c ln(floor((p + 1) / every) + 1);
               s_ij = cap * tanh(scale * q_i.k_j / cap) + rel[bucket(i - j), head];  softmax over j <= i;  W_o
  bucket(n)    n if n < B/2 else min(B - 1, B/2 + floor(ln(n / (B/2)) / ln(D / (B/2)) * (B - B/2)))
  delta        q, k, v = silu(causal conv_taps(W h));  q, k to unit length (1e-6 in the root), q *= dim^-1/2;
               beta = sigmoid(W_b h);  g = exp(-exp(A_log) softplus(W_a h + dt_bias));
               S = g S;  u = beta (v - S^T k);  S += k u^T;  o = S^T q;  out = W_o (rms(o) * w * silu(W_g h))
  moe          mean over the token's table row of W_down (silu(W_gate h) * (W_up h))
  side         y = W_proj (gelu_tanh(W_gate x) * side_embed[token, layer slice]);  y / sqrt(mean(y^2) + eps) * w
"""
import math

import numpy as np


def _np(t):
    return t.detach().to("cpu").double().numpy() if hasattr(t, "detach") else np.asarray(t, dtype=np.float64)


def rms(y, eps):
    return y / np.sqrt(np.mean(y * y, axis=-1, keepdims=True) + eps)


def silu(z):
    return z / (1.0 + np.exp(-z))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z):
    return np.log1p(np.exp(-np.abs(z))) + np.maximum(z, 0.0)


def bucket(n, nb, reach):
    half = nb // 2
    if n < half:
        return n
    return min(nb - 1, half + int(math.floor(math.log(n / half) / math.log(reach / half) * (nb - half))))


def project_kv(w, pre, mc, h, eps):
    t = h.shape[0]
    k = rms((h @ _np(w[pre + "k"]).T).reshape(t, mc["kv_heads"], mc["dim"]), eps)
    v = rms((h @ _np(w[pre + "v"]).T).reshape(t, mc["kv_heads"], mc["vdim"]), eps)
    return k, v


def attention(w, pre, mc, h, eps, kv):
    t = h.shape[0]
    nh, ng, d, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    q = rms((h @ _np(w[pre + "q"]).T).reshape(t, nh, d), eps)
    if "q_temp" in mc:
        for p in range(t):
            q[p] *= 1.0 + mc["q_temp"]["coef"] * math.log((p + 1) // mc["q_temp"]["every"] + 1)
    k, v = kv
    rel = _np(w[pre + "rel"]) if pre + "rel" in w else None
    out = np.zeros((t, nh, dv))
    for head in range(nh):
        g = head // (nh // ng)
        for i in range(t):
            s = np.empty(i + 1)
            for j in range(i + 1):
                x = float(q[i, head] @ k[j, g]) * mc["scale"]
                if mc.get("softcap"):
                    x = mc["softcap"] * math.tanh(x / mc["softcap"])
                if rel is not None:
                    x += rel[bucket(i - j, rel.shape[0], mc["bias_max"]), head]
                s[j] = x
            pr = np.exp(s - s.max())
            pr /= pr.sum()
            out[i, head] = pr @ v[: i + 1, g]
    return out.reshape(t, nh * dv) @ _np(w[pre + "o"]).T


def short_conv_silu(x, cw):
    t, taps = x.shape[0], cw.shape[1]
    y = np.zeros_like(x)
    for i in range(t):
        for tap in range(taps):
            src = i - (taps - 1) + tap
            if src >= 0:
                y[i] += cw[:, tap] * x[src]
    return silu(y)


def delta(w, pre, mc, h, eps):
    t = h.shape[0]
    nh, ng, d, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    q = short_conv_silu(h @ _np(w[pre + "q"]).T, _np(w[pre + "q.conv"])).reshape(t, ng, d)
    k = short_conv_silu(h @ _np(w[pre + "k"]).T, _np(w[pre + "k.conv"])).reshape(t, ng, d)
    v = short_conv_silu(h @ _np(w[pre + "v"]).T, _np(w[pre + "v.conv"])).reshape(t, nh, dv)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * d ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = 1.0 / (1.0 + np.exp(-(h @ _np(w[pre + "b"]).T)))
    g = np.exp(-np.exp(_np(w[pre + "A_log"])) * softplus(h @ _np(w[pre + "a"]).T + _np(w[pre + "dt_bias"])))
    o = np.zeros((t, nh, dv))
    for head in range(nh):
        kh = head // (nh // ng)
        state = np.zeros((d, dv))
        for i in range(t):
            state = g[i, head] * state
            u = beta[i, head] * (v[i, head] - state.T @ k[i, kh])
            state = state + np.outer(k[i, kh], u)
            o[i, head] = state.T @ q[i, kh]
    o = rms(o, eps) * _np(w[pre + "norm"])
    return (o.reshape(t, nh * dv) * silu(h @ _np(w[pre + "g"]).T)) @ _np(w[pre + "o"]).T


def moe(w, pre, fc, h, tokens):
    top = fc["router"]["top"]
    table = np.asarray(w[pre + "table"])
    out = np.zeros_like(h)
    for i, tok in enumerate(tokens):
        for c in range(top):
            e = int(table[tok, c])
            p = f"{pre}e{e}."
            out[i] += _np(w[p + "down"]) @ (silu(_np(w[p + "gate"]) @ h[i]) * (_np(w[p + "up"]) @ h[i])) / top
    return out


def side_input(w, pre, i, sd, x, tokens, eps):
    e = _np(w["side.embed"])[tokens][:, i * sd:(i + 1) * sd]
    y = (gelu_tanh(x @ _np(w[pre + "gate"]).T) * e) @ _np(w[pre + "proj"]).T
    return rms(y, eps) * _np(w[pre + "norm"])


def forward(cfg, w, tokens):
    """``(logits [T, V], hidden [layers, T, width])`` of one sequence, float64."""
    tokens = [int(t) for t in tokens]
    eps = cfg["norm"]["eps"]
    x = _np(w["embed"])[tokens]
    hidden, kvs = [], {}
    for i, layer in enumerate(cfg["layers"]):
        pre, mc = f"l{i}.", layer["mixer"]
        if layer["type"] == "attention":
            src = mc.get("kv_from")
            kvs[i] = kvs[src] if src is not None else project_kv(w, pre + "mix.", mc, x, eps)
            y = attention(w, pre + "mix.", mc, x, eps, kvs[i])
        else:
            y = delta(w, pre + "mix.", mc, x, eps)
        x = x + rms(y, eps) * float(_np(w[pre + "norm1"]))
        if layer.get("mlp") is not None:
            x = x + rms(moe(w, pre + "mlp.", layer["mlp"], x, tokens), eps) * float(_np(w[pre + "norm2"]))
        if cfg.get("token_side"):
            x = x + side_input(w, pre + "side.", i, cfg["token_side"]["dim"], x, tokens, eps)
        hidden.append(x.copy())
    logits = (rms(x, eps) * float(_np(w["final.norm"]))) @ _np(w["head"]).T
    return logits, np.stack(hidden)
