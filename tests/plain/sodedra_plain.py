"""Plain, slow Sodedra forward pass: whole sequences, no cache, one function per mechanism.

Sodedra is a decoder whose layers read ONE norm of the stream with both sublayers and add their
sum (``x + mixer(n(x)) + ff(n(x))``, the norm's weight stored around zero).  A layer's token
mixer is one of three: a matrix memory with exponential input gate and a running maximum
(mLSTM), a grouped-query attention with projection biases, partly rotated heads (frequencies
rescaled by wavelength), a sliding window and a sigmoid gate on its output, or a gated delta
rule with short causal convolutions and a decay per key channel.  The feed-forward is a gated
dense layer or a mixture of such experts whose router picks among the best groups of experts.
The embedding is scaled, and the output head is the unscaled embedding table.

This file shares no code with the ``spyinfer_amd`` package.  It takes a configuration as a
dictionary and the tensors as a dictionary of CPU tensors, and computes in ``dtype``
(float64 by default).
"""
import json
import math
import os

import torch


# ---- pieces ------------------------------------------------------------------------------
def rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def zero_centred_norm(x, w, eps):
    return rms(x, eps) * (1.0 + w)


def silu(z):
    return z * torch.sigmoid(z)


def gated_ff(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def route(z, correction, top, groups, keep, scale):
    """Router logits z [T, E] -> (chosen experts [T, top], their weights [T, top])."""
    T, E = z.shape
    s = torch.softmax(z, dim=-1)
    choice = s + correction
    per = E // groups
    best = choice.view(T, groups, per).max(dim=-1).values
    kept = torch.topk(best, keep, dim=-1).indices
    allowed = torch.zeros((T, groups), dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    masked = torch.where(allowed[:, :, None].expand(T, groups, per).reshape(T, E), choice,
                         torch.full_like(choice, -math.inf))
    ids = torch.topk(masked, top, dim=-1).indices
    w = torch.gather(s, 1, ids)
    w = w / (w.sum(dim=-1, keepdim=True) + 1e-20) * scale
    return ids, w


def moe_ff(h, w, router):
    """w: the layer's 'mlp.*' tensors by short name; router: the configuration's numbers."""
    E = router["experts"]
    ids, wt = route(h @ w["router"].T, w["correction"], router["top"], router["groups"]["count"], router["groups"]["keep"],
                    router["scale"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            e = int(ids[t, j])
            assert 0 <= e < E
            out[t] += wt[t, j] * gated_ff(h[t:t + 1], w["e%d.gate" % e], w["e%d.up" % e], w["e%d.down" % e])[0]
    return out


def scaled_frequencies(dims, base, scaling, dtype=torch.float64):
    """f_i = base^(-2i/dims); by wavelength l = 2 pi / f: short ones stay, long ones are divided by the factor, those
    between are blended."""
    i = torch.arange(dims // 2, dtype=dtype)
    f = torch.tensor(float(base), dtype=dtype) ** (-2.0 * i / dims)
    if not scaling:
        return f
    factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = f.clone()
    for j in range(dims // 2):
        wl = 2.0 * math.pi / float(f[j])
        if wl < original / high:
            continue
        if wl > original / low:
            out[j] = f[j] / factor
        else:
            s = (original / wl - low) / (high - low)
            out[j] = (1.0 - s) * f[j] / factor + s * f[j]
    return out


def rotate_half(x, positions, freq, dims):
    """x [T, heads, n]: the first ``dims`` entries of a head are rotated, pair (i, i + dims/2); the rest pass."""
    half = dims // 2
    ang = positions.to(freq.dtype)[:, None] * freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


def gated_attention(h, w, m):
    """h [T, width]; w: the mixer's tensors by short name; m: its configuration."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T + w["q.b"]).view(T, H, d)
    k = (h @ w["k"].T + w["k.b"]).view(T, G, d)
    v = (h @ w["v"].T + w["v.b"]).view(T, G, dv)
    rot = m.get("rot")
    if rot:
        pos = torch.arange(T)
        f = scaled_frequencies(rot["dims"], rot["base"], rot.get("scaling"), h.dtype)
        q, k = rotate_half(q, pos, f, rot["dims"]), rotate_half(k, pos, f, rot["dims"])
    window = m["mask"]["size"] if m.get("mask") else None
    out = torch.zeros((T, H, dv), dtype=h.dtype)
    for i in range(T):
        lo = 0 if window is None else max(0, i - window + 1)
        for hd in range(H):
            g = hd // (H // G)
            sc = (k[lo:i + 1, g] @ q[i, hd]) * m["scale"]
            out[i, hd] = torch.softmax(sc, dim=0) @ v[lo:i + 1, g]
    out = out.reshape(T, H * dv) * torch.sigmoid(h @ w["g"].T)
    return out @ w["o"].T


def capped(z, cap):
    return cap * torch.tanh(z / cap)


def mlstm(h, w, m, eps):
    """Matrix memory per head, S [dim, vdim] and n [dim] with a running maximum m of the log gates (starting at 0)."""
    T = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = (h @ w["q"].T).view(T, H, d) * d ** -0.5
    k = (h @ w["k"].T).view(T, H, d)
    v = (h @ w["v"].T).view(T, H, dv)
    ig = capped(h @ w["i"].T + w["i.b"], cap)
    fg = torch.nn.functional.logsigmoid(capped(h @ w["f"].T + w["f.b"], cap))
    out = torch.zeros((T, H, dv), dtype=h.dtype)
    for hd in range(H):
        S = torch.zeros((d, dv), dtype=h.dtype)
        n = torch.zeros((d,), dtype=h.dtype)
        mx = 0.0
        for t in range(T):
            new = max(float(fg[t, hd]) + mx, float(ig[t, hd]))
            a, b = math.exp(float(fg[t, hd]) + mx - new), math.exp(float(ig[t, hd]) - new)
            S = a * S + b * torch.outer(k[t, hd], v[t, hd])
            n = a * n + b * k[t, hd]
            mx = new
            den = max(abs(float(n @ q[t, hd])), math.exp(-mx)) + 1e-6
            out[t, hd] = (S.T @ q[t, hd]) / den
    out = rms(out, eps).reshape(T, H * dv) * w["norm"] * torch.sigmoid(h @ w["g"].T)
    return out @ w["o"].T


def causal_conv(x, taps):
    """x [T, C], taps [C, n]: y[t] = sum_j taps[:, j] x[t - (n - 1) + j], zeros before the start."""
    T, n = x.shape[0], taps.shape[1]
    pad = torch.cat([torch.zeros((n - 1, x.shape[1]), dtype=x.dtype), x], dim=0)
    return sum(pad[j:j + T] * taps[:, j] for j in range(n))


def unit(x):
    return x / torch.sqrt((x * x).sum(dim=-1, keepdim=True) + 1e-6)


def channel_delta(h, w, m, eps):
    """Gated delta rule per head with a decay per key channel."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit(silu(causal_conv(h @ w["q"].T, w["q.conv"])).view(T, G, d)) * d ** -0.5
    k = unit(silu(causal_conv(h @ w["k"].T, w["k.conv"])).view(T, G, d))
    v = silu(causal_conv(h @ w["v"].T, w["v.conv"])).view(T, H, dv)
    beta = torch.sigmoid(h @ w["b"].T)
    dt = torch.nn.functional.softplus((h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]).view(T, H, d)
    decay = torch.exp(-torch.exp(w["A_log"])[None, :, None] * dt)
    out = torch.zeros((T, H, dv), dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros((d, dv), dtype=h.dtype)
        for t in range(T):
            S = decay[t, hd][:, None] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, hd] = S.T @ q[t, g]
    gate = torch.sigmoid((h @ w["g1"].T) @ w["g2"].T).view(T, H, dv)
    out = (rms(out, eps) * w["norm"] * gate).reshape(T, H * dv)
    return out @ w["o"].T


# ---- the model ---------------------------------------------------------------------------
class PlainSodedra:
    def __init__(self, config, tensors, dtype=torch.float64):
        self.cfg = config
        self.w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
        self.dtype = dtype

    @classmethod
    def from_folder(cls, folder, dtype=torch.float64):
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        return cls(cfg, load_file(os.path.join(folder, "model.safetensors")), dtype)

    def sub(self, prefix):
        return {k[len(prefix):]: v for k, v in self.w.items() if k.startswith(prefix)}

    def forward(self, tokens, keep_layers=None):
        """Logits [T, vocab] at every position of one sequence; ``keep_layers``: a list that gets the stream after
        every layer."""
        cfg, eps = self.cfg, float(self.cfg["norm"]["eps"])
        x = self.w["embed"][torch.tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
        for i, layer in enumerate(cfg["layers"]):
            h = zero_centred_norm(x, self.w["l%d.norm1" % i], eps)
            mw = self.sub("l%d.mix." % i)
            if layer["type"] == "mlstm":
                y = mlstm(h, mw, layer["mixer"], eps)
            elif layer["type"] == "attention":
                y = gated_attention(h, mw, layer["mixer"])
            elif layer["type"] == "channel_delta":
                y = channel_delta(h, mw, layer["mixer"], eps)
            else:
                raise ValueError(layer["type"])
            mlp = layer.get("mlp")
            if mlp:
                fw = self.sub("l%d.mlp." % i)
                y = y + (gated_ff(h, fw["gate"], fw["up"], fw["down"]) if mlp["kind"] == "dense" else moe_ff(h, fw, mlp["router"]))
            x = x + y
            if keep_layers is not None:
                keep_layers.append(x.clone())
        return zero_centred_norm(x, self.w["final.norm"], eps) @ self.w["embed"].T

    def greedy(self, prompt, n):
        toks = list(prompt)
        for _ in range(n):
            toks.append(int(torch.argmax(self.forward(toks)[-1])))
        return toks[len(prompt):]
