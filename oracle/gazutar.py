"""Plain, slow statement of the Gazutar design (torch on CPU, float64 by default): one function per mechanism.

TEST INFRASTRUCTURE: nothing of the product path imports this file and it imports nothing of the product path.
It processes one sequence at a time, whole, with dense [T, T] score matrices and a Python loop over time for the
recurrent layers - the thing the paged, batched, chunked kernels are compared against.

Notation (W x means `x @ W.T`, weights are stored [out, in]):

  layer         x <- x + LN1(mixer(x));  x <- x + LN2(ff(x))      (the norm sits on the sublayer's OUTPUT)
  LN            (y - mean(y)) / sqrt(var(y) + eps) * w + b,  var = mean of squared deviations
  attention     q = rms_all(W_q h) * w_qn, k = rms_all(W_k h) * w_kn   (ONE root mean square over the whole projection)
                s_ij = scale * q_i . k_j - slope_h * (i - j),  slope_h = 2^(-8 (h + 1) / H),  0 <= i - j < window
                p = softmax_j(s),  o_i = sum_j p_ij v_j,  out = W_o (o * sigmoid(W_g h))
                v <- (1 - lam) v + lam v_first in every value-mixing layer but the first one
  channel_delta per head: S <- diag(g_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
                q, k, v after a short causal depthwise convolution and silu; q, k unit vectors, q / sqrt(dim)
                g = exp(-exp(A_log_h) softplus(W_a2 W_a1 h + dt_bias)),  beta = sigmoid(W_b h)
                out = W_o (rms_head(o) * w_norm * sigmoid(W_g2 W_g1 h))
  ff            sparse mixture: scores = softmax(W_r h) over experts + identity experts, choice = scores + correction,
                choice restricted to the best `keep` of `count` groups (a group's score = its largest choice score),
                top-k of choice; weights = the chosen SCORES, not renormalised; identity experts return h
  output        logits = logit_scale * W_head LN_final(x)
"""
from __future__ import annotations

import math

import torch


def layer_norm(y, w, b, eps):
    mu = y.mean(-1, keepdim=True)
    var = ((y - mu) ** 2).mean(-1, keepdim=True)
    return (y - mu) / torch.sqrt(var + eps) * w + b


def rms_all(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def slopes(n_heads, dtype):
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / n_heads) for h in range(n_heads)], dtype=dtype)


def windowed_attention(q, k, v, scale, window):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] of one sequence -> [T, H, Dv]; dense scores, -inf outside the window."""
    T, H, _ = q.shape
    G = k.shape[1]
    dist = torch.arange(T).view(T, 1) - torch.arange(T).view(1, T)
    visible = (dist >= 0) & (dist < window)
    sl = slopes(H, q.dtype)
    out = torch.empty(T, H, v.shape[-1], dtype=q.dtype)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * scale - sl[hd] * dist.to(q.dtype)
        out[:, hd] = torch.softmax(s.masked_fill(~visible, float("-inf")), -1) @ v[:, g]
    return out


def attention_mixer(h, p, cfg, eps, v_first, is_first_vmix):
    """h [T, W] of ONE sequence -> (mixer output [T, W], this layer's values as cached [T, G * vdim])."""
    T = h.shape[0]
    H, G, D, Dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    q = rms_all(h @ p["q"].T, p["q.norm"], eps).view(T, H, D)
    k = rms_all(h @ p["k"].T, p["k.norm"], eps).view(T, G, D)
    v = h @ p["v"].T
    if cfg.get("v_mix") and not is_first_vmix:
        lam = p["vmix"]
        v = (1 - lam) * v + lam * v_first
    out = windowed_attention(q, k, v.view(T, G, Dv), cfg["scale"], cfg["mask"]["size"])
    gate = torch.sigmoid(h @ p["g"].T)
    return (out.reshape(T, H * Dv) * gate) @ p["o"].T, v


def causal_conv(x, w):
    """x [T, C], w [C, taps] (last column multiplies the current token), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    xp = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], 0)
    y = torch.zeros_like(x)
    for t in range(taps):
        y = y + xp[t:t + T] * w[:, t]
    return y


def channel_delta_mixer(h, p, cfg, eps):
    T = h.shape[0]
    H, G, D, Dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    q = silu(causal_conv(h @ p["q"].T, p["q.conv"])).view(T, G, D)
    k = silu(causal_conv(h @ p["k"].T, p["k.conv"])).view(T, G, D)
    v = silu(causal_conv(h @ p["v"].T, p["v.conv"])).view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ p["b"].T)                                   # [T, H]
    dt = torch.nn.functional.softplus((h @ p["a1"].T) @ p["a2"].T + p["dt_bias"]).view(T, H, D)
    g = torch.exp(-torch.exp(p["A_log"]).view(1, H, 1) * dt)              # [T, H, D]
    o = torch.empty(T, H, Dv, dtype=h.dtype)
    for hd in range(H):
        kv = hd // (H // G)
        S = torch.zeros(D, Dv, dtype=h.dtype)
        for t in range(T):
            S = g[t, hd].view(D, 1) * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kv])
            S = S + torch.outer(k[t, kv], u)
            o[t, hd] = S.T @ q[t, kv]
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * p["norm"]
    gate = torch.sigmoid((h @ p["g1"].T) @ p["g2"].T).view(T, H, Dv)
    return (o * gate).reshape(T, H * Dv) @ p["o"].T


def route(h, p, cfg):
    """-> (ids [T, top] , weights [T, top]); ids >= experts name identity experts."""
    r = cfg["router"]
    n = r["experts"] + r.get("identity", 0)
    z = h @ p["router"].T
    s = torch.softmax(z, -1)
    choice = s + p["correction"]
    cnt, keep = r["groups"]["count"], r["groups"]["keep"]
    per = n // cnt
    gscore = choice.view(-1, cnt, per).max(-1).values
    kept = torch.zeros_like(gscore, dtype=torch.bool)
    kept.scatter_(1, gscore.topk(keep, -1).indices, True)
    choice = choice.masked_fill(~kept.repeat_interleave(per, 1), float("-inf"))
    ids = choice.topk(r["top"], -1).indices
    return ids, s.gather(1, ids)


def moe(h, p, cfg):
    ids, wts = route(h, p, cfg)
    E = cfg["router"]["experts"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(ids[t].tolist(), wts[t]):
            if e >= E:
                out[t] += w * h[t]
            else:
                y = silu(h[t] @ p[f"e{e}.gate"].T) * (h[t] @ p[f"e{e}.up"].T)
                out[t] += w * (y @ p[f"e{e}.down"].T)
    return out


def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(config, weights, tokens, dtype=torch.float64, collect=None):
    """Logits [T, vocab] of one whole sequence.  collect: a list that receives the residual stream after every layer."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens)]
    v_first = None
    for i, layer in enumerate(config["layers"]):
        pre = f"l{i}."
        mix = sub(W, pre + "mix.")
        if layer["type"] == "attention":
            first = layer["mixer"].get("v_mix") and v_first is None
            y, v = attention_mixer(x, mix, layer["mixer"], eps, v_first, first)
            if first:
                v_first = v
        elif layer["type"] == "channel_delta":
            y = channel_delta_mixer(x, mix, layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + layer_norm(y, W[pre + "norm1"], W[pre + "norm1.b"], eps)
        if layer.get("mlp") is not None:
            y = moe(x, sub(W, pre + "mlp."), layer["mlp"])
            x = x + layer_norm(y, W[pre + "norm2"], W[pre + "norm2.b"], eps)
        if collect is not None:
            collect.append(x.clone())
    x = layer_norm(x, W["final.norm"], W["final.norm.b"], eps)
    return (x @ W["head"].T) * config["logit_scale"]


def random_model(config, seed=0, scale=None):
    """Random bf16-representable weights for a config of this design (names and shapes as a checkpoint has them)."""
    g = torch.Generator().manual_seed(seed)
    Wd, V = config["width"], config["vocab"]

    def mat(o, i, s=None):
        return (torch.randn(o, i, generator=g) * (s if s is not None else i ** -0.5)).bfloat16().float()

    def vec(n, mean=0.0, s=0.1):
        return (mean + torch.randn(n, generator=g) * s).bfloat16().float()

    w = {"embed": mat(V, Wd, 1.0), "head": mat(V, Wd), "final.norm": vec(Wd, 1.0), "final.norm.b": vec(Wd)}
    for i, layer in enumerate(config["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        for n in ("norm1", "norm2"):
            w[pre + n], w[pre + n + ".b"] = vec(Wd, 1.0), vec(Wd)
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        if layer["type"] == "attention":
            w[pre + "mix.q"], w[pre + "mix.k"], w[pre + "mix.v"] = mat(H * D, Wd), mat(G * D, Wd), mat(G * Dv, Wd)
            w[pre + "mix.q.norm"], w[pre + "mix.k.norm"] = vec(H * D, 1.0), vec(G * D, 1.0)
            if m.get("v_mix"):
                w[pre + "mix.vmix"] = vec(1, 0.4)[0]
            w[pre + "mix.g"], w[pre + "mix.o"] = mat(H * Dv, Wd), mat(Wd, H * Dv)
        else:
            r = m.get("rank", max(8, Wd // 8))
            w[pre + "mix.q"], w[pre + "mix.k"], w[pre + "mix.v"] = mat(G * D, Wd), mat(G * D, Wd), mat(H * Dv, Wd)
            for n, c in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                w[pre + f"mix.{n}.conv"] = mat(c, m["conv"], 0.6)
            w[pre + "mix.b"], w[pre + "mix.A_log"], w[pre + "mix.norm"] = mat(H, Wd), vec(H, -1.0, 0.5), vec(Dv, 1.0)
            w[pre + "mix.a1"], w[pre + "mix.a2"], w[pre + "mix.dt_bias"] = mat(r, Wd), mat(H * D, r), vec(H * D, -1.0, 1.0)
            w[pre + "mix.g1"], w[pre + "mix.g2"], w[pre + "mix.o"] = mat(r, Wd), mat(H * Dv, r), mat(Wd, H * Dv)
        if layer.get("mlp") is not None:
            ml = layer["mlp"]
            E, ff = ml["router"]["experts"], ml["expert"]["ff"]
            n = E + ml["router"].get("identity", 0)
            for e in range(E):
                w[pre + f"mlp.e{e}.gate"], w[pre + f"mlp.e{e}.up"] = mat(ff, Wd), mat(ff, Wd)
                w[pre + f"mlp.e{e}.down"] = mat(Wd, ff)
            w[pre + "mlp.router"], w[pre + "mlp.correction"] = mat(n, Wd, 2.0 * Wd ** -0.5), vec(n, 0.0, 0.05)
    return w
