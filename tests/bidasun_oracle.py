"""Plain, slow oracle of the Bidasun design for the tests: one function per mechanism, written
from the design's equations in float64, whole sequences at a time, no cache, no batching. It
shares no code with nv_genai_amd (it does not import it)."""
import math

import torch

F64 = torch.float64


def o_rms(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def o_gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def o_embed(tokens, embed, pos_table):
    """Token row plus the learned row of the position (positions count from 0)."""
    return torch.stack([embed[t] + pos_table[p] for p, t in enumerate(tokens)])


def o_token_shift(x, mu):
    """h_t = x_t + (x_{t-1} - x_t) * mu, with x_{-1} = 0."""
    out = torch.empty_like(x)
    for t in range(x.shape[0]):
        prev = x[t - 1] if t > 0 else torch.zeros_like(x[0])
        out[t] = x[t] + (prev - x[t]) * mu
    return out


def o_visible(i, j, window, keep_first):
    return j <= i and (i - j < window or j < keep_first)


def o_sigmoid_attention(q, k, v, heads, kv_heads, scale, window, keep_first, r1, r2, pb):
    """q [T, heads, dk], k [T, kv_heads, dk], v [T, kv_heads, dv] -> [T, heads, dv]. Weight of a
    visible key: sigmoid(q.k * scale - r1 ln(1 + r2 (i - j)) + pb); weights are not normalised."""
    T = q.shape[0]
    out = torch.zeros(T, heads, v.shape[-1], dtype=q.dtype)
    group = heads // kv_heads
    for i in range(T):
        js = torch.tensor([j for j in range(T) if o_visible(i, j, window, keep_first)])
        dist = (i - js).to(q.dtype)
        for h in range(heads):
            g = h // group
            s = (k[js, g] @ q[i, h]) * scale - r1[h] * torch.log1p(r2[h] * dist)
            wgt = 1.0 / (1.0 + torch.exp(-(s + pb[h])))
            out[i, h] = wgt @ v[js, g]
    return out


def o_mixer(h, W, p, m, eps):
    """The attention mixer of block prefix ``p`` with sizes ``m`` (a config.json mixer dict)."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = o_rms(h @ W[p + "mix.q"].T, W[p + "mix.q.norm"], eps).view(T, H, dk)
    k = o_rms(h @ W[p + "mix.k"].T, W[p + "mix.k.norm"], eps).view(T, G, dk)
    v = (h @ W[p + "mix.v"].T).view(T, G, dv)
    a = o_sigmoid_attention(q, k, v, H, G, m["scale"], m["mask"]["size"], m["mask"]["keep_first"],
                            W[p + "mix.r1"], W[p + "mix.r2"], W[p + "mix.pb"])
    a = a.reshape(T, H * dv) * torch.sigmoid(h @ W[p + "mix.g"].T)
    return a @ W[p + "mix.o"].T


def o_mlp(x, W, p):
    return (o_gelu_tanh(x @ W[p + "mlp.gate"].T) * (x @ W[p + "mlp.up"].T)) @ W[p + "mlp.down"].T


def o_forward(cfg, W, tokens):
    """cfg: the config.json dict; W: name -> float64 tensor. Returns (logits [T, vocab], the
    residual stream after every block [layers, T, width])."""
    eps = cfg["norm"]["eps"]
    x = o_embed(tokens, W["embed"], W["pos"])
    after = []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = o_token_shift(x, W[p + "shift"])
        x = x + o_rms(o_mixer(h, W, p, L["mixer"], eps), W[p + "norm1"], eps)
        if L["mlp"] is not None:
            x = x + o_rms(o_mlp(x, W, p), W[p + "norm2"], eps)
        after.append(x.clone())
    return o_rms(x, W["final.norm"], eps) @ W["head"].T, torch.stack(after)


def o_greedy(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(o_forward(cfg, W, toks)[0][-1].argmax()))
    return toks[len(prompt):]
