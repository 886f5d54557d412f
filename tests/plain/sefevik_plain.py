"""Plain, slow Sefevik forward pass: whole sequences, no cache, one function per mechanism.

Sefevik is a decoder whose layers add the RMS norm of a sublayer's output to the stream
(``x + norm(f(x))``, the sublayer reading ``x`` itself), mix the results of all earlier layers
with learned weights before the next layer, and take their token mixer from two kinds: a
minimal gated recurrence and a latent attention (keys and values expanded from one low-rank
vector per token, a rotated key part shared by the heads, a sliding window and a per-head sink
in the softmax).  The embedding adds a hashed row for the pair (previous token, token).

This file shares no code with the ``spyinfer_amd`` package.  It takes a configuration as a
dictionary and the tensors as a dictionary of CPU tensors, and computes in ``dtype``
(float64 by default).
"""
import json
import math
import os

import torch


# ---- pieces ------------------------------------------------------------------------------
def rms_norm(x, w, eps):
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def softplus(x):
    return math.log1p(math.exp(-abs(x))) + max(x, 0.0)


def xielu(z, p, q):
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (e^z - 1 - z) + z/2."""
    ap, aq = softplus(float(p)), 0.5 + softplus(float(q))
    pos = ap * z * z + 0.5 * z
    neg = aq * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def dense_ff(h, up, down, act):
    return xielu(h @ up.T, act[0], act[1]) @ down.T


def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the pair table for every token: a hash of (previous, current); the first token takes the last row."""
    rows = []
    for i, t in enumerate(tokens):
        rows.append(buckets if i == 0 else (tokens[i - 1] * mul_prev + t * mul_cur) % buckets)
    return rows


def yarn_frequencies(dims, base, scaling, dtype=torch.float64):
    """(frequencies [dims/2], factor on cos and sin)."""
    half = dims // 2
    i = torch.arange(half, dtype=dtype)
    f = torch.tensor(float(base), dtype=dtype) ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def corr(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(corr(float(scaling["fast"]))), 0)
    hi = min(math.ceil(corr(float(scaling["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half(x, positions, freq, mag, dims):
    """x [..., T, n]: the first ``dims`` entries are rotated, pair (i, i + dims/2); the rest pass."""
    half = dims // 2
    ang = positions.to(freq.dtype)[:, None] * freq[None, :]
    c, s = torch.cos(ang) * mag, torch.sin(ang) * mag
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


def min_gru(h, w, state=None):
    """h [T, width_in]; w: z, z.b, x, x.b, g, o.  Returns (out [T, width_in], last state)."""
    z = torch.sigmoid(h @ w["z"].T + w["z.b"])
    u = h @ w["x"].T + w["x.b"]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    gate = h @ w["g"].T
    s = torch.zeros(z.shape[1], dtype=h.dtype) if state is None else state
    out = []
    for t in range(h.shape[0]):
        s = (1.0 - z[t]) * s + z[t] * cand[t]
        out.append(s * (gate[t] * torch.sigmoid(gate[t])))
    return torch.stack(out) @ w["o"].T, s


def latent_kv(h, w, m, eps, positions):
    """What a latent-attention layer caches per token: (latent [T, kv_rank], rotated shared key part [T, rot_dim])."""
    r = m["kv_rank"]
    d = h @ w["dkv"].T
    c = rms_norm(d[:, :r], w["dkv.norm"], eps)
    rot = m.get("rot") or {}
    dims = rot.get("dims", m["rot_dim"])
    freq, mag = yarn_frequencies(dims, rot["base"], rot.get("scaling"), h.dtype) if rot else (None, 1.0)
    kr = rotate_half(d[:, r:], positions, freq, mag, dims) if rot else d[:, r:]
    return c, kr


def latent_attention(h, w, m, positions, c, kr):
    """h [T, width]; c, kr as ``latent_kv`` gives them (this layer's or another's)."""
    T = h.shape[0]
    H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    q = (h @ w["q"].T).view(T, H, dn + dr)
    rot = m.get("rot") or {}
    if rot:
        dims = rot.get("dims", dr)
        freq, mag = yarn_frequencies(dims, rot["base"], rot.get("scaling"), h.dtype)
        q_rot = rotate_half(q[:, :, dn:].transpose(0, 1), positions, freq, mag, dims).transpose(0, 1)
    else:
        q_rot = q[:, :, dn:]
    k = (c @ w["uk"].T).view(T, H, dn)
    v = (c @ w["uv"].T).view(T, H, dv)
    scores = (torch.einsum("thd,jhd->htj", q[:, :, :dn], k) + torch.einsum("thd,jd->htj", q_rot, kr)) * float(m["scale"])
    i, j = positions[:, None], positions[None, :]
    seen = (j <= i)
    window = (m.get("mask") or {}).get("size")
    if window is not None:
        seen = seen & (i - j < window)
    scores = scores.masked_fill(~seen[None], float("-inf"))
    sink = w["sink"].to(h.dtype)[:, None, None].expand(H, T, 1)
    p = torch.softmax(torch.cat([scores, sink], dim=-1), dim=-1)[..., :-1]      # the sink has no value
    out = torch.einsum("htj,jhd->thd", p, v).reshape(T, H * dv)
    return out @ w["o"].T


# ---- the model ---------------------------------------------------------------------------
class PlainSefevik:
    def __init__(self, config, tensors, dtype=torch.float64):
        self.cfg, self.dtype = config, dtype
        self.w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}

    @classmethod
    def from_folder(cls, folder, dtype=torch.float64):
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        return cls(cfg, load_file(os.path.join(folder, "model.safetensors")), dtype)

    def sub(self, prefix):
        n = len(prefix)
        return {k[n:]: v for k, v in self.w.items() if k.startswith(prefix)}

    def embed(self, tokens):
        x = self.w["embed"][torch.tensor(tokens)]
        bg = (self.cfg.get("embedding") or {}).get("bigram")
        if bg:
            x = x + self.w["bigram"][torch.tensor(bigram_rows(tokens, bg["buckets"], bg["mul_prev"], bg["mul_cur"]))]
        return x

    def forward(self, tokens, layers_out=None):
        """Logits [T, vocab] of one sequence from its start.  ``layers_out``: a list that receives what every layer
        hands on."""
        cfg, eps = self.cfg, float(self.cfg["norm"]["eps"])
        pos = torch.arange(len(tokens))
        x = self.embed(tokens)
        results = [x]
        kept = {}
        for i, layer in enumerate(cfg["layers"]):
            m, pre = layer["mixer"], "l%d." % i
            mix = self.sub(pre + "mix.")
            if layer["type"] == "mingru":
                y, _ = min_gru(x, mix)
            elif layer["type"] == "latent_attention":
                src = m.get("kv_from")
                if src is None:
                    kept[i] = latent_kv(x, mix, m, eps, pos)
                    src = i
                y = latent_attention(x, mix, m, pos, *kept[src])
            else:
                raise ValueError(layer["type"])
            x = x + rms_norm(y, self.w[pre + "norm1"], eps)
            if layer.get("mlp"):
                ff = self.sub(pre + "mlp.")
                x = x + rms_norm(dense_ff(x, ff["up"], ff["down"], ff["act"]), self.w[pre + "norm2"], eps)
            results.append(x)
            if pre + "dwa" in self.w:
                a = self.w[pre + "dwa"]
                x = sum(a[j] * results[j] for j in range(len(results)))
            if layers_out is not None:
                layers_out.append(x)
        return rms_norm(x, self.w["final.norm"], eps) @ self.w["head"].T

    def greedy(self, prompt, n):
        toks = list(prompt)
        for _ in range(n):
            toks.append(int(torch.argmax(self.forward(toks)[-1])))
        return toks[len(prompt):]
