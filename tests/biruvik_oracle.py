"""Plain float64 implementation of the Biruvik decoder, one function per mechanism, whole
sequences, no cache, no batching. It imports nothing from the package: the tests compare the
serving path against it.

Notation: ``x`` [T, width] residual rows of one sequence, positions 0 .. T-1; weights are a dict
of float64 tensors under the checkpoint's tensor names; ``cfg`` is the config.json dict.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm with one gain for all coordinates."""
    return rms(x, eps) * g


def relu2_ff(h, w, p):
    u = torch.relu(h @ w[p + "mlp.up"].T)
    return (u * u) @ w[p + "mlp.down"].T


def q_temperature(T, coef, every):
    """Per-position query factor 1 + coef * ln(floor((p + 1) / every) + 1)."""
    p = torch.arange(T, dtype=F64)
    return 1.0 + coef * torch.log(torch.floor((p + 1) / every) + 1.0)


def softmax_rows(scores, visible):
    s = scores.masked_fill(~visible, float("-inf"))
    s = s - s.max(-1, keepdim=True).values
    e = torch.exp(s)
    return e / e.sum(-1, keepdim=True)


def causal_mask(T, window=0):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    m = j <= i
    if window:
        m = m & (i - j < window)
    return m


def differential_attention(h, w, p, m, eps):
    """Two softmax maps per head over shared values: o = a1 - lam * a2, unit RMS per head,
    times (1 - diff). GQA; per head-and-map RMS norm of q and k; query temperature; no rotation."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "mix.q"].T + w[p + "mix.q.b"]).view(T, H, 2, d)
    k = (h @ w[p + "mix.k"].T + w[p + "mix.k.b"]).view(T, G, 2, d)
    v = (h @ w[p + "mix.v"].T + w[p + "mix.v.b"]).view(T, G, dv)
    q = rms(q, eps) * w[p + "mix.q.norm"]
    k = rms(k, eps) * w[p + "mix.k.norm"]
    q = q * q_temperature(T, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None, None, None]
    lam = (math.exp(float((w[p + "mix.lq1"] * w[p + "mix.lk1"]).sum()))
           - math.exp(float((w[p + "mix.lq2"] * w[p + "mix.lk2"]).sum())) + m["diff"])
    vis = causal_mask(T)
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        a = []
        for mp in range(2):
            s = (q[:, hh, mp] @ k[:, g, mp].T) * m["scale"]
            a.append(softmax_rows(s, vis) @ v[:, g])
        o = a[0] - lam * a[1]
        out[:, hh] = rms(o, eps) * (1.0 - m["diff"])
    return out.reshape(T, H * dv) @ w[p + "mix.o"].T


def latent_attention(h, w, p, m, eps):
    """Keys and values expanded from one normalised latent per token; sliding window; sigmoid
    output gate per head; no positions."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "mix.q"].T).view(T, H, d)
    c = rms(h @ w[p + "mix.dkv"].T, eps) * w[p + "mix.dkv.norm"]
    k = (c @ w[p + "mix.uk"].T).view(T, H, d)
    v = (c @ w[p + "mix.uv"].T).view(T, H, dv)
    gate = torch.sigmoid(h @ w[p + "mix.g"].T)
    vis = causal_mask(T, m["mask"]["size"])
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        s = (q[:, hh] @ k[:, hh].T) * m["scale"]
        out[:, hh] = (softmax_rows(s, vis) @ v[:, hh]) * gate[:, hh:hh + 1]
    return out.reshape(T, H * dv) @ w[p + "mix.o"].T


def hgrn2(h, w, p, m, eps):
    """Gated linear recurrence: the forget gate f decays the state rows and 1 - f writes them."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = torch.nn.functional.silu(h @ w[p + "mix.q"].T).view(T, H, d)
    v = (h @ w[p + "mix.v"].T).view(T, H, dv)
    low = w[p + "mix.lower"]
    f = (low + (1.0 - low) * torch.sigmoid(h @ w[p + "mix.f"].T + w[p + "mix.f.b"])).view(T, H, d)
    S = torch.zeros(H, d, dv, dtype=F64)
    out = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    out = rms(out, eps) * w[p + "mix.norm"]
    return out.reshape(T, H * dv) @ w[p + "mix.o"].T


MIXERS = {"attention": differential_attention, "latent_attention": latent_attention, "hgrn2": hgrn2}


def forward(cfg: dict, weights: dict, tokens, layer_tap=None):
    """Logits [T, vocab] of one whole sequence (float64)."""
    w = {k: v.to(F64) for k, v in weights.items() if v.dtype.is_floating_point}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        o = MIXERS[L["type"]](scalar_norm(x, w[p + "norm1"], eps), w, p, L["mixer"], eps)
        x = x + scalar_norm(o, w[p + "norm1b"], eps)
        if L.get("mlp") is not None:
            o = relu2_ff(scalar_norm(x, w[p + "norm2"], eps), w, p)
            x = x + scalar_norm(o, w[p + "norm2b"], eps)
        if layer_tap is not None:
            layer_tap.append(x.clone())
    z = scalar_norm(x, w["final.norm"], eps) @ w["head"].T
    cap = cfg["logit_softcap"]
    return cap * torch.tanh(z / cap)


def greedy(cfg: dict, weights: dict, prompt, n: int):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, weights, toks)[-1].argmax()))
    return toks[len(prompt):]
