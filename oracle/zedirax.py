"""Plain, slow statement of the Zedirax design (torch on CPU, float64 by default): one function per mechanism.

TEST INFRASTRUCTURE: nothing of the product path imports this file and it imports nothing of the product path.
One sequence at a time, whole, with dense [T, T] score matrices and a Python loop over time for the recurrence.

Notation (W x means `x @ W.T`, weights stored [out, in]; p = position, counted from 0):

  norm          n(x; w) = x / sqrt(mean(x^2) + eps) * (1 + w)           (the weight is stored around zero)
  layer i       a <- a + m * mixer(n1(a));  a <- a + m * ff(n2(a));  X_{i+1} = a
                the next layer (and the output) reads  sum_{j <= i+1} d_i[j] X_j   (X_0: the embedding rows)
  mingru        z = sigmoid(W_z h + b_z), u = W_x h + b_x, c = u + 1/2 (u >= 0) | sigmoid(u) (u < 0)
                S_p = (1 - z) S_{p-1} + z c,  S_{-1} = 0;   out = W_o (S_p * silu(W_g h))
  latent_attn   [c | r] = W_dkv h;  c <- c / rms(c) * w_c  (plain weight);  r, and the last `rot_dim` entries of every
                query head, are rotated by p;  k_h = [W_uk,h c | r],  v_h = W_uv,h c
                s = scale * q_h . k_h,  causal softmax;  out = W_o (concat_h(o_h) * sigmoid(W_g h))
  rotation      the first `dims` entries of the rotated part: pairs (i, i + dims/2), angle p * base^(-2 i / dims)
  attention     q_p <- q_p * (1 + coef * ln(floor((p + 1) / every) + 1))
                s_ij = scale * q_i . k_j - r1_h * ln(1 + r2_h (i - j)),  causal softmax, grouped key/value heads
  dense ff      W_d (gelu_tanh(W_g h + b_g) * (W_u h + b_u)) + b_d
  sparse ff     logits = W_r h;  the `top` largest;  weights = softmax over the chosen logits
                out = sum_k w_k W_d,e gelu_erf(W_u,e h)  +  sigmoid(w_sg . h) * W_d,s gelu_erf(W_u,s h)
  output        logits = W_head n(x; w_final)
"""
from __future__ import annotations

import math

import torch


def rms_norm(x, w, eps, centred: bool):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y * (1 + w) if centred else y * w


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def gelu_erf(z):
    return 0.5 * z * (1 + torch.erf(z / math.sqrt(2.0)))


def silu(z):
    return z * torch.sigmoid(z)


def rotate(x, pos, dims, base):
    """x [T, ..., R]: the first `dims` entries of the last axis turn by pos * base^(-2 i / dims), halves paired."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    ang = pos.to(x.dtype).view(-1, *([1] * (x.dim() - 2)), 1) * f
    c, s = torch.cos(ang), torch.sin(ang)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def causal_softmax_attention(scores, v):
    """scores [H, T, T] (already biased), v [T, H, Dv] -> [T, H, Dv]"""
    T = scores.shape[-1]
    hidden = torch.arange(T).view(1, T) > torch.arange(T).view(T, 1)
    p = torch.softmax(scores.masked_fill(hidden, float("-inf")), -1)
    return torch.einsum("hij,jhd->ihd", p, v)


def mingru_mixer(h, p):
    z = torch.sigmoid(h @ p["z"].T + p["z.b"])
    u = h @ p["x"].T + p["x.b"]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    S = torch.zeros(z.shape[1], dtype=h.dtype)
    states = []
    for t in range(h.shape[0]):
        S = (1 - z[t]) * S + z[t] * cand[t]
        states.append(S)
    return (torch.stack(states) * silu(h @ p["g"].T)) @ p["o"].T


def latent_attention_mixer(h, p, m, eps):
    T = h.shape[0]
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (h @ p["q"].T).view(T, H, D + R)
    dkv = h @ p["dkv"].T
    c = rms_norm(dkv[:, :C], p["dkv.norm"], eps, centred=False)
    dims, base = int(m["rot"]["dims"]), float(m["rot"]["base"])
    r = rotate(dkv[:, C:], pos, dims, base)
    q_rot = rotate(q[..., D:], pos, dims, base)
    k = (c @ p["uk"].T).view(T, H, D)
    v = (c @ p["uv"].T).view(T, H, Dv)
    s = (torch.einsum("ihd,jhd->hij", q[..., :D], k) + torch.einsum("ihd,jd->hij", q_rot, r)) * m["scale"]
    o = causal_softmax_attention(s, v).reshape(T, H * Dv)
    return (o * torch.sigmoid(h @ p["g"].T)) @ p["o"].T


def biased_attention_mixer(h, p, m):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (h @ p["q"].T).view(T, H, D)
    qt = m.get("q_temp")
    if qt:
        temp = 1 + qt["coef"] * torch.log(torch.floor((pos + 1) / qt["every"]).to(h.dtype) + 1)
        q = q * temp.view(T, 1, 1)
    k = (h @ p["k"].T).view(T, G, D).repeat_interleave(H // G, 1)
    v = (h @ p["v"].T).view(T, G, Dv).repeat_interleave(H // G, 1)
    dist = (pos.view(T, 1) - pos.view(1, T)).clamp(min=0).to(h.dtype)
    bias = p["r1"].view(H, 1, 1) * torch.log(1 + p["r2"].view(H, 1, 1) * dist)
    s = torch.einsum("ihd,jhd->hij", q, k) * m["scale"] - bias
    return causal_softmax_attention(s, v).reshape(T, H * Dv) @ p["o"].T


def dense_ff(h, p):
    return (gelu_tanh(h @ p["gate"].T + p["gate.b"]) * (h @ p["up"].T + p["up.b"])) @ p["down"].T + p["down.b"]


def small_ff(h, p, prefix):
    return gelu_erf(h @ p[prefix + "up"].T) @ p[prefix + "down"].T


def sparse_ff(h, p, ml):
    top = int(ml["router"]["top"])
    logits = h @ p["router"].T
    val, idx = torch.topk(logits, top, dim=-1)
    w = torch.softmax(val, -1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for k in range(top):
            out[t] += w[t, k] * small_ff(h[t:t + 1], p, f"e{int(idx[t, k])}.")[0]
    if ml.get("shared"):
        out = out + torch.sigmoid(h @ p["shared.sg"].T) * small_ff(h, p, "shared.")
    return out


def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(config, weights, tokens, dtype=torch.float64, collect=None):
    """Logits [T, vocab] of one sequence; `collect` (a list) receives what every layer hands on."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps, m = float(config["norm"]["eps"]), float(config["residual_mult"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    results = [x]
    for i, spec in enumerate(config["layers"]):
        p = sub(w, f"l{i}.")
        h = rms_norm(x, p["norm1"], eps, centred=True)
        mp = sub(p, "mix.")
        if spec["type"] == "mingru":
            y = mingru_mixer(h, mp)
        elif spec["type"] == "latent_attention":
            y = latent_attention_mixer(h, mp, spec["mixer"], eps)
        elif spec["type"] == "attention":
            y = biased_attention_mixer(h, mp, spec["mixer"])
        else:
            raise ValueError(spec["type"])
        x = x + m * y
        ml = spec.get("mlp")
        if ml is not None:
            h = rms_norm(x, p["norm2"], eps, centred=True)
            x = x + m * (dense_ff(h, sub(p, "mlp.")) if ml["kind"] == "dense" else sparse_ff(h, sub(p, "mlp."), ml))
        results.append(x)
        x = sum(p["dwa"][j] * results[j] for j in range(i + 2))
        if collect is not None:
            collect.append(x)
    return rms_norm(x, w["final.norm"], eps, centred=True) @ w["head"].T


def tensor_shapes(config):
    """name -> shape of a checkpoint of this configuration"""
    W, V = int(config["width"]), int(config["vocab"])
    out = {"embed": (V, W), "head": (V, W), "final.norm": (W,)}
    for i, spec in enumerate(config["layers"]):
        pre, m = f"l{i}.", spec["mixer"]
        out[pre + "norm1"] = (W,)
        out[pre + "dwa"] = (i + 2,)
        if spec["type"] == "mingru":
            n = int(m["width"])
            out.update({pre + "mix.z": (n, W), pre + "mix.z.b": (n,), pre + "mix.x": (n, W), pre + "mix.x.b": (n,),
                        pre + "mix.g": (n, W), pre + "mix.o": (W, n)})
        elif spec["type"] == "latent_attention":
            H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            out.update({pre + "mix.q": (H * (D + R), W), pre + "mix.dkv": (C + R, W), pre + "mix.dkv.norm": (C,),
                        pre + "mix.uk": (H * D, C), pre + "mix.uv": (H * Dv, C), pre + "mix.g": (H * Dv, W),
                        pre + "mix.o": (W, H * Dv)})
        else:
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({pre + "mix.q": (H * D, W), pre + "mix.k": (G * D, W), pre + "mix.v": (G * Dv, W),
                        pre + "mix.r1": (H,), pre + "mix.r2": (H,), pre + "mix.o": (W, H * Dv)})
        ml = spec.get("mlp")
        if ml is None:
            continue
        out[pre + "norm2"] = (W,)
        if ml["kind"] == "dense":
            F = int(ml["ff"])
            out.update({pre + "mlp.gate": (F, W), pre + "mlp.gate.b": (F,), pre + "mlp.up": (F, W), pre + "mlp.up.b": (F,),
                        pre + "mlp.down": (W, F), pre + "mlp.down.b": (W,)})
        else:
            F = int(ml["expert"]["ff"])
            out[pre + "mlp.router"] = (int(ml["router"]["experts"]), W)
            for e in range(int(ml["router"]["experts"])):
                out[pre + f"mlp.e{e}.up"] = (F, W)
                out[pre + f"mlp.e{e}.down"] = (W, F)
            if ml.get("shared"):
                Fs = int(ml["shared"]["ff"])
                out.update({pre + "mlp.shared.up": (Fs, W), pre + "mlp.shared.down": (W, Fs), pre + "mlp.shared.sg": (1, W)})
    return out


def random_model(config, seed=0, overrides=None):
    """Random bf16-representable weights (so that a bf16 checkpoint of them is exact) under the checkpoint's names."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        leaf = name.rsplit(".", 1)[-1]
        if name.endswith("norm1") or name.endswith("norm2") or name == "final.norm":
            t = torch.randn(shape, generator=g) * 0.1
        elif name.endswith("dkv.norm"):
            t = 1 + torch.randn(shape, generator=g) * 0.1
        elif leaf == "dwa":
            t = torch.randn(shape, generator=g) * 0.15
            t[-1] += 1.0
        elif leaf == "r1":
            t = torch.rand(shape, generator=g) * 1.5 + 0.1
        elif leaf == "r2":
            t = torch.rand(shape, generator=g) * 2.0 + 0.05
        elif leaf == "b":
            t = torch.randn(shape, generator=g) * 0.3
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * (1.5 * shape[-1] ** -0.5)
        out[name] = t.to(torch.bfloat16).to(torch.float32)
    for k, v in (overrides or {}).items():
        out[k] = v.to(torch.bfloat16).to(torch.float32)
    return out
