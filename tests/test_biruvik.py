"""Biruvik on the serving engine against the plain oracle (tests/biruvik_oracle.py).

Every case runs on the CPU (the engine on the fp32 reference ops: scheduling, pages, state
slots, row maps) and, marked ``gpu``, on the HIP kernels in float32 and bfloat16. The models are
small random ones built here; sizes are chosen so that heads, kv heads, dim, vdim, ranks, windows
and the page size do not coincide (``odd``), or so that the MFMA tile kernels run (``tiles``).
"""
import json
import math

import pytest
import torch

import biruvik_oracle as O
from nv_genai_amd import ops
from nv_genai_amd.engine.llm_engine import EngineConfig, LLMEngine, SamplingParams
from nv_genai_amd.models.biruvik import BiruvikModel, random_weights
from nv_genai_amd.models.config import BiruvikConfig

GPU = pytest.param("cuda", marks=pytest.mark.gpu)
DEVICES = ["cpu", GPU]
DTYPES = [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu),
          pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu)]


def attn(heads=3, kv_heads=1, dim=8, vdim=12, scale=0.3, diff=0.2, coef=0.4, every=50, ff=24):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                           "scale": scale, "diff": diff, "q_temp": {"coef": coef, "every": every}},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def latent(heads=5, dim=8, vdim=4, kv_rank=20, scale=0.25, window=70, ff=24):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank,
                                                  "scale": scale, "mask": {"size": window}},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def hgrn(heads=3, dim=12, vdim=20, ff=24):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def cfg_dict(layers, width=40, vocab=97, eps=1e-5, scale=7.0, cap=25.0):
    return {"architecture": "Biruvik", "vocab": vocab, "width": width, "embedding": {"scale": scale},
            "norm": {"eps": eps}, "logit_softcap": cap, "layers": layers}


def cfg_odd():
    return cfg_dict([hgrn(), attn(heads=4, kv_heads=2), latent(), attn(heads=2, kv_heads=2, dim=12, vdim=8, ff=None),
                     latent(heads=2, dim=4, vdim=12, kv_rank=9, window=9, ff=None), hgrn(heads=1, dim=5, vdim=70)])


def cfg_tiles():
    """Head sizes the MFMA kernels take (multiples of 32), unequal per layer."""
    return cfg_dict([attn(heads=4, kv_heads=2, dim=64, vdim=32, scale=0.12), latent(heads=3, dim=16, vdim=32, kv_rank=64),
                     hgrn(heads=2, dim=32, vdim=64),
                     attn(heads=2, kv_heads=1, dim=32, vdim=128, scale=0.18, every=64, ff=None),
                     latent(heads=18, dim=16, vdim=16, kv_rank=128, window=130, scale=0.2)], width=48)


CFGS = {"odd": cfg_odd, "tiles": cfg_tiles}


def build(device, dtype="float32", seed=0, pages=24, seqs=4, cd=None, graphs=None, **eng):
    cd = cd or cfg_odd()
    cfg = BiruvikConfig.from_dict(cd)
    w = random_weights(cfg, seed, torch.bfloat16)       # bf16 values, as a checkpoint holds them
    tdt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    model = BiruvikModel(cfg, device, tdt, weights=w)
    kw = dict(model="biruvik-test", dtype=dtype, max_num_seqs=seqs, max_batched_tokens=512, max_model_len=512,
              kv_cache_blocks=pages, detokenize=False, use_graphs=(device == "cuda") if graphs is None else graphs,
              graph_batch_sizes=(1, 2, 4), mixed_graphs=False, logits_tap=True, tuned_gemms=False, async_decode=False)
    kw.update(eng)
    e = LLMEngine(EngineConfig(**kw), device=device, model=model)
    return e, cd, w


def tokens(n, vocab=97, seed=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def tol(dtype):
    return 2e-4 if dtype == "float32" else 6e-2


def close(got, want, dtype, what=""):
    got, want = got.double().cpu(), want.double()
    err = (got - want).abs().max().item() / max(1.0, want.abs().max().item())
    assert err < tol(dtype), f"{what}: relative error {err:.3e}"


def replay_cuts(eng, toks, cuts, rid=1, finish=True):
    """Feed ``toks`` in portions of the given sizes (the rest one token at a time); all logits."""
    out, at, cuts = [], 0, list(cuts)
    while at < len(toks):
        n = min(cuts.pop(0) if cuts else 1, len(toks) - at)
        done = at + n == len(toks)
        out.append(eng.replay_step([(rid, toks[at:at + n], list(range(n)))], [rid] if done and finish else []))
        at += n
    return torch.cat(out)


# ---------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_sandwich_norms_embedding_relu2_softcap(device, dtype):
    torch.manual_seed(1)
    tdt = getattr(torch, dtype)
    for H in (36, 300):
        x, y = torch.randn(7, H), torch.randn(7, H).to(tdt)
        for w, nw in ((torch.tensor([0.7]), torch.tensor([1.3])), (torch.rand(H) + 0.5, torch.rand(H) + 0.5)):
            xd = x.clone().to(device)
            h = ops.rmsnorm_residual_next_(xd, y.to(device), w.to(device), 1e-5, nw.to(device), tdt)
            want = x.double() + O.rms(y.double(), 1e-5) * w.double()
            close(xd, want, "float32", "residual sum")
            close(h, O.rms(want, 1e-5) * nw.double(), dtype, "next norm")
    table = torch.randn(11, 20).to(tdt)
    ids = torch.tensor([3, 0, 10, 3], dtype=torch.int32)
    close(ops.embed_rows(ids.to(device), table.to(device), 12.5), table.double()[ids.long()] * 12.5, "float32", "embedding")
    for n in (35, 64):
        u = torch.randn(3, n).to(tdt)
        close(ops.relu_sq(u.to(device)), torch.relu(u.double()) ** 2, dtype, "relu squared")
    z = torch.randn(5, 33) * 40
    close(ops.softcap_(z.clone().to(device), 30.0), 30.0 * torch.tanh(z.double() / 30.0), "float32", "soft cap")
    o = torch.randn(6, 3 * 20)
    gw = torch.rand(20) + 0.5
    close(ops.group_rmsnorm(o.to(device), gw.to(device), 3, 1e-5, tdt),
          (O.rms(o.double().view(6, 3, 20), 1e-5) * gw.double()).reshape(6, 60), dtype, "head norm")


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_head_norm_temperature_and_cache_write(device, dtype):
    torch.manual_seed(2)
    tdt = getattr(torch, dtype)
    for nq, nk, dk, nv, dv, pad in ((6, 2, 8, 1, 12, 5), (4, 4, 32, 2, 64, 0), (0, 1, 20, 0, 0, 7)):
        T = 70
        n0, n1, n2 = nq * dk, (nq + nk) * dk, (nq + nk) * dk + nv * dv
        proj = torch.randn(T, n2 + pad).to(tdt)
        qw, kw, bias = torch.rand(dk) + 0.5, torch.rand(dk) + 0.5, torch.randn(n2) * 0.3
        bt = [5, 2]
        slots = torch.tensor([bt[t // 64] * 64 + t % 64 for t in range(T)], dtype=torch.int32)
        slots[3] = -1                                       # a row that writes nothing
        pos = torch.arange(100, 100 + T, dtype=torch.int32)  # positions cross multiples of `every`
        kc = torch.zeros(6, max(nk, 1), 64, dk, dtype=tdt, device=device)
        vc = torch.zeros(6, nv, 64, dv, dtype=tdt, device=device) if nv else None
        p64 = proj.double()
        b64 = bias.double()
        pd = proj.clone().to(device)
        ops.headnorm_cache_(pd, slots.to(device), kc, vc, nq, nk, dk, nv, dv, 1e-5, q_w=qw.to(device) if nq else None,
                            k_w=kw.to(device), bias=bias.to(device), pos=pos.to(device), temp_coef=0.4 if nq else 0.0,
                            temp_every=13)
        kn = (O.rms((p64[:, n0:n1] + b64[n0:n1]).view(T, nk, dk), 1e-5) * kw.double())
        vn = p64[:, n1:n2] + b64[n1:n2]
        if nq:
            temp = 1.0 + 0.4 * torch.log(torch.floor((pos.double() + 1) / 13) + 1.0)
            qn = O.rms((p64[:, :n0] + b64[:n0]).view(T, nq, dk), 1e-5) * qw.double() * temp[:, None, None]
            close(pd[:, :n0], qn.reshape(T, n0), dtype, "q: bias, head norm, temperature")
            want_t = O.q_temperature(T + 100, 0.4, 13)[100:]
            assert torch.allclose(temp, want_t)
        close(pd[:, n0:n1], kn.reshape(T, -1), dtype, "k in place")
        for t in (0, 63, 64, 69):
            close(kc[bt[t // 64], :, t % 64, :], kn[t], dtype, f"k page row {t}")
            if nv:
                close(vc[bt[t // 64], :, t % 64, :], vn[t].view(nv, dv), dtype, f"v page row {t}")
        assert kc[bt[0], :, 3].abs().sum() == 0
        if pad:
            close(pd[:, n2:], p64[:, n2:], dtype, "columns past q | k | v untouched")


def _paged(k, v, device, tdt, bt_row, nb=None):
    """k [T, Gk, dk], v [T, Gv, dv] into row-major pages listed by bt_row."""
    T, Gk, dk = k.shape
    nb = nb or max(bt_row) + 1
    kc = torch.zeros(nb, Gk, 64, dk, dtype=tdt, device=device)
    vc = torch.zeros(nb, v.shape[1], 64, v.shape[2], dtype=tdt, device=device)
    for t in range(T):
        kc[bt_row[t // 64], :, t % 64, :] = k[t].to(tdt).to(device)
        vc[bt_row[t // 64], :, t % 64, :] = v[t].to(tdt).to(device)
    return kc, vc


def o_softmax_attention(q, k, v, H, G, scale, window, maps, lam, unit_eps, out_scale, gate):
    """Oracle: q [T, H, maps, dk], k [T, G, maps, dk], v [T, G, dv] (float64), whole sequence."""
    T = q.shape[0]
    vis = O.causal_mask(T, window)
    out = torch.zeros(T, H, v.shape[-1], dtype=O.F64)
    for h in range(H):
        g = h // (H // G)
        a = [O.softmax_rows((q[:, h, m] @ k[:, g, m].T) * scale, vis) @ v[:, g] for m in range(maps)]
        o = a[0] - lam * a[1] if maps == 2 else a[0]
        if unit_eps is not None:
            o = O.rms(o, unit_eps) * out_scale
        if gate is not None:
            o = o * torch.sigmoid(gate[:, h:h + 1])
        out[:, h] = o
    return out.reshape(T, -1)


ATTN_SHAPES = [  # H, G, dk, dv, window, maps
    (4, 2, 8, 12, 0, 2), (5, 1, 20, 20, 70, 1), (3, 3, 8, 8, 9, 1), (1, 1, 4, 4, 1, 2),
    (4, 2, 32, 64, 0, 2), (18, 1, 64, 64, 130, 1), (2, 1, 64, 32, 64, 2), (3, 1, 128, 128, 100, 1)]


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_softmax_attention_random(device, dtype):
    torch.manual_seed(3)
    tdt = getattr(torch, dtype)
    for H, G, dk, dv, W, maps in ATTN_SHAPES:
        T = 150
        q = torch.randn(T, H, maps, dk).to(tdt)
        k, v = torch.randn(T, G, maps, dk).to(tdt), torch.randn(T, G, dv).to(tdt)
        gate = torch.randn(T, H).to(tdt) if maps == 1 else None
        ue = 1e-5 if maps == 2 else None
        bt_row = [4, 0, 7]
        kc, vc = _paged(k.reshape(T, G * maps, dk), v, device, tdt, bt_row)
        bt = torch.tensor([[9, 9, 9], bt_row], dtype=torch.int32, device=device)
        want = o_softmax_attention(q.double(), k.double(), v.double(), H, G, 0.3, W, maps, 0.45, ue, 0.8,
                                   None if gate is None else gate.double())
        pos = torch.arange(T, dtype=torch.int32, device=device)
        seq = torch.ones(T, dtype=torch.int32, device=device)
        kw = dict(window=W, maps=maps, lam=0.45, unit_eps=ue, out_scale=0.8)
        gd = None if gate is None else gate.to(device)
        got = ops.softmax_attention(q.reshape(T, -1).to(device), kc, vc, bt, seq, pos, H, G, dk, dv, 0.3, gate=gd, **kw)
        close(got, want, dtype, f"attention {H},{G},{dk},{dv},{W},{maps}")
        # the same rows one at a time, shuffled, as decode rows of a batch would come
        order = torch.randperm(T)[:40]
        got1 = ops.softmax_attention_rows(q.reshape(T, -1)[order].contiguous().to(device), kc, vc, bt, seq[:40],
                                          pos[order.to(device)].contiguous(), H, G, dk, dv, 0.3, max_ctx=192,
                                          gate=None if gd is None else gd[order.to(device)].contiguous(), **kw)
        close(got1, want[order], dtype, f"single rows {H},{G},{dk},{dv},{W},{maps}")


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_one_key_stands_out(device, dtype):
    """One key scores far above the rest (q and that key scaled up): the softmax output is that
    key's value when the key is visible; when it is not, the output is the mean of the visible
    values (all other scores are equal). Keys far back, at page borders and at both sides of the
    window's edge, as the end of a prompt portion and as a single row, through the row kernel,
    the prompt kernel and the single-token kernel."""
    tdt = getattr(torch, dtype)
    T = 200
    bt_row = [3, 1, 6, 2]
    bt = torch.tensor([bt_row], dtype=torch.int32, device=device)
    for H, dk, dv, W in ((1, 32, 32, 37), (2, 8, 12, 0), (1, 64, 64, 64), (1, 32, 64, 65)):
        for i in (199, 128, 127, 64, 63, 40, 36, 1, 0):
            cands = {0, i - W - 1, i - W, i - W + 1, i - 1, i, 63, 64, 127, 128, i // 2}
            for j in sorted(c for c in cands if 0 <= c <= i):
                k = torch.zeros(T, 1, dk)
                k[j, 0, 0] = 8.0
                v = torch.randn(T, 1, dv)
                q = torch.zeros(T, H, dk)
                q[:, :, 0] = 8.0                              # q.k = 64 for key j, 0 for the rest
                kc, vc = _paged(k, v, device, tdt, bt_row)
                lo = max(0, i - W + 1) if W else 0
                vis = lo <= j <= i
                v64 = v[:, 0].to(tdt).double()
                want = v64[j] if vis else v64[lo:i + 1].mean(0)
                for rows in (list(range(max(0, i - 2), i + 1)), [i]):     # a portion ending at i / i alone
                    pos = torch.tensor(rows, dtype=torch.int32, device=device)
                    seq = torch.zeros(len(rows), dtype=torch.int32, device=device)
                    qr = q.reshape(T, -1)[rows].contiguous().to(tdt).to(device)
                    args = (H, 1, dk, dv, 1.0)
                    outs = {"row kernel": ops.softmax_attention(qr, kc, vc, bt, seq, pos, *args, window=W),
                            "single-token kernel": ops.softmax_attention_rows(qr, kc, vc, bt, seq, pos, *args,
                                                                              max_ctx=256, window=W)}
                    if len(rows) > 1:
                        cu = torch.tensor([0, len(rows)], dtype=torch.int32, device=device)
                        cx = torch.tensor([i + 1], dtype=torch.int32, device=device)
                        outs["prompt kernel"] = ops.softmax_attention_prefill(qr, kc, vc, bt, cu, cx, len(rows), *args,
                                                                              window=W)
                    for name, got in outs.items():
                        err = (got[-1].double().cpu().view(H, dv) - want).abs().max().item()
                        assert err < 2e-2, f"{name}: query {i}, key {j}, window {W}, visible {vis}: off by {err}"


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_softmax_attention_prompt_portions(device, dtype):
    """The prompt-portion entry point (MFMA tiles for bf16 on the GPU): three sequences whose
    portions start in the middle of a page, end past a window and differ in length."""
    torch.manual_seed(4)
    tdt = getattr(torch, dtype)
    for H, G, dk, dv, W, maps in ATTN_SHAPES[4:] + ATTN_SHAPES[:2]:
        ctxs, qlens = [200, 67, 130], [150, 67, 2]
        bts = [[4, 0, 7, 9], [1, 2, 11, 11], [3, 5, 6, 11]]
        nb = 12
        kc = torch.zeros(nb, G * maps, 64, dk, dtype=tdt, device=device)
        vc = torch.zeros(nb, G, 64, dv, dtype=tdt, device=device)
        ue = 1e-5 if maps == 2 else None
        qs, gs, wants = [], [], []
        for c, n, bt_row in zip(ctxs, qlens, bts):
            q = torch.randn(c, H, maps, dk).to(tdt)
            k, v = torch.randn(c, G, maps, dk).to(tdt), torch.randn(c, G, dv).to(tdt)
            gate = torch.randn(c, H).to(tdt)
            for t in range(c):
                kc[bt_row[t // 64], :, t % 64, :] = k[t].reshape(G * maps, dk).to(device)
                vc[bt_row[t // 64], :, t % 64, :] = v[t].to(device)
            want = o_softmax_attention(q.double(), k.double(), v.double(), H, G, 0.2, W, maps, 0.3, ue, 0.75,
                                       gate.double())
            qs.append(q.reshape(c, -1)[c - n:])
            gs.append(gate[c - n:])
            wants.append(want[c - n:])
        cu = torch.tensor([0, 150, 217, 219], dtype=torch.int32, device=device)
        btd = torch.tensor(bts, dtype=torch.int32, device=device)
        kw = dict(window=W, maps=maps, lam=0.3, unit_eps=ue, out_scale=0.75)
        got = ops.softmax_attention_prefill(torch.cat(qs).to(device), kc, vc, btd, cu,
                                            torch.tensor(ctxs, dtype=torch.int32, device=device), 150, H, G, dk, dv,
                                            0.2, gate=torch.cat(gs).to(device), **kw)
        close(got, torch.cat(wants), dtype, f"prompt portions {H},{G},{dk},{dv},{W},{maps}")
        seq = torch.tensor([0] * 150 + [1] * 67 + [2] * 2, dtype=torch.int32, device=device)
        pos = torch.cat([torch.arange(c - n, c) for c, n in zip(ctxs, qlens)]).int().to(device)
        pick = torch.tensor([0, 13, 149, 150, 216, 217, 218, 77], device=device)
        got1 = ops.softmax_attention_rows(torch.cat(qs).to(device)[pick].contiguous(), kc, vc, btd, seq[pick].contiguous(),
                                          pos[pick].contiguous(), H, G, dk, dv, 0.2, max_ctx=256,
                                          gate=torch.cat(gs).to(device)[pick].contiguous(), **kw)
        close(got1, torch.cat(wants)[pick.cpu()], dtype, f"single-token rows {H},{G},{dk},{dv},{W},{maps}")


def o_hgrn2_raw(qp, fp, v, fb, low):
    """Oracle of the recurrence alone: pre-activations [T, H, d] / [T, H, dv] -> un-normalised o."""
    T, H, d = qp.shape
    q = torch.nn.functional.silu(qp)
    f = low + (1 - low) * torch.sigmoid(fp + fb)
    S = torch.zeros(H, d, v.shape[-1], dtype=O.F64)
    out = []
    for t in range(T):
        S = f[t][:, :, None] * S + (1 - f[t])[:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hdv,hd->hv", S, q[t]))
    return torch.stack(out), S


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_hgrn2_scan_segments_and_slots(device, dtype):
    """Two sequences in portions (one of a single row, one of 19, one that starts in the middle)
    and as single rows, with a slot that held another sequence before."""
    torch.manual_seed(5)
    tdt = getattr(torch, dtype)
    for H, d, dv in ((3, 12, 20), (2, 32, 64), (1, 5, 70), (2, 70, 8), (1, 140, 32)):
        T = 40
        raw = [torch.randn(T, 2 * H * d + H * dv + 3).to(tdt) for _ in range(2)]
        fb, low = torch.randn(H * d) * 0.5, torch.rand(H * d) * 0.9
        wants = []
        for r in raw:
            r64 = r.double()
            o, S = o_hgrn2_raw(r64[:, :H * d].view(T, H, d), r64[:, H * d:2 * H * d].view(T, H, d),
                               r64[:, 2 * H * d:2 * H * d + H * dv].reshape(T, H, dv), fb.double().view(H, d),
                               low.double().view(H, d))
            wants.append((o.reshape(T, -1), S))
        state = torch.randn(3, H, d, dv, device=device)      # stale contents: position 0 must not read them
        slots = torch.tensor([2, 0], dtype=torch.int32, device=device)
        got = [[], []]
        at = [0, 0]
        for step in ([1, 19], [19, 2], [5, 0], [15, 19]):
            rows = torch.cat([raw[b][at[b]:at[b] + n] for b, n in enumerate(step)]).to(device)
            pos = torch.cat([torch.arange(at[b], at[b] + n) for b, n in enumerate(step)]).int().to(device)
            cu = torch.tensor([0, step[0], step[0] + step[1]], dtype=torch.int32, device=device)
            o = ops.hgrn2_scan(rows, fb.to(device), low.to(device), state, H, d, dv, cu, slots, pos)
            got[0].append(o[:step[0]])
            got[1].append(o[step[0]:])
            at = [a + n for a, n in zip(at, step)]
        for b in range(2):
            close(torch.cat(got[b]), wants[b][0], "float32" if dtype == "float32" else dtype, f"portions {H},{d},{dv}")
            close(state[int(slots[b])], wants[b][1], "float32" if dtype == "float32" else dtype, "state after the last row")
        # single rows (cu = None), a slot of -1 reads and keeps nothing
        st2 = torch.randn(3, H, d, dv, device=device)
        keep = st2[1].clone()
        outs = []
        for t in range(6):
            rows = torch.stack([raw[0][t], raw[1][t], raw[1][t]]).to(device)
            pos = torch.tensor([t, t, t], dtype=torch.int32, device=device)
            outs.append(ops.hgrn2_scan(rows, fb.to(device), low.to(device), st2, H, d, dv, None,
                                       torch.tensor([0, 2, -1], dtype=torch.int32, device=device), pos))
        for b in range(2):
            close(torch.stack([o[b] for o in outs]), wants[b][0][:6], dtype, "single rows")
        close(outs[0][2], wants[1][0][0], dtype, "row without a slot at position 0")
        assert torch.equal(st2[1], keep)


# ---------------------------------------------------------------------------- the model on the engine
@pytest.mark.parametrize("shape", sorted(CFGS))
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_whole_prompt_and_layers(device, dtype, shape):
    eng, cd, W = build(device, dtype, cd=CFGS[shape]())
    toks = tokens(200)
    layers = []
    want = O.forward(cd, W, toks, layers)
    tap = []
    got = eng.replay_step([(1, toks, list(range(len(toks))))], [1], layer_tap=tap)
    for i, (a, b) in enumerate(zip(tap, layers)):
        close(a, b, dtype, f"residual stream after layer {i} ({cd['layers'][i]['type']})")
    close(got, want, dtype, "logits")
    close(got[:3], O.forward(cd, W, toks[:3]), dtype, "first tokens")
    close(eng.replay_step([(2, toks[:1], [0])], [2]), O.forward(cd, W, toks[:1]), dtype, "a prompt of one token")


@pytest.mark.parametrize("shape", sorted(CFGS))
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_prefill_then_decode_and_portions(device, dtype, shape):
    eng, cd, W = build(device, dtype, cd=CFGS[shape]())
    toks = tokens(230, seed=5)
    want = O.forward(cd, W, toks)
    close(replay_cuts(eng, toks, [70]), want, dtype, "prompt then token by token (160 decoded, windows pass)")
    close(replay_cuts(eng, toks, [1] * 3 + [2, 61, 2, 3, 64, 2, 63, 2, 17]), want, dtype, "portions down to two tokens")
    close(replay_cuts(eng, toks, []), want, dtype, "token by token from the first")
    assert eng.sched.free_blocks() == eng.num_blocks and eng.sched.free_state_slots() == 4


@pytest.mark.parametrize("shape", sorted(CFGS))
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_mixed_batches_and_reuse(device, dtype, shape):
    """Unequal requests interleaved (portions beside single tokens, a request that skips steps),
    in a pool that only holds the live ones: pages and slots are freed and used again by requests
    that start later. Every request must equal its run alone (the oracle)."""
    eng, cd, W = build(device, dtype, pages=9, seqs=3, cd=CFGS[shape]())
    reqs = {i: tokens(n, seed=10 + i) for i, n in enumerate((150, 65, 1, 200, 129, 64, 3))}
    want = {i: O.forward(cd, W, t) for i, t in reqs.items()}
    got = {i: [] for i in reqs}
    at = {i: 0 for i in reqs}
    waiting, live, step = sorted(reqs), [], 0
    plans = {0: [64, 1, 1, 30], 1: [2, 62], 3: [100, 2], 4: [128], 5: [63]}
    while waiting or live:
        while waiting and len(live) < 3:
            nxt = waiting[0]
            need = sum(-(-len(reqs[i]) // 64) for i in live) + -(-len(reqs[nxt]) // 64)
            if need > 9:
                break
            live.append(waiting.pop(0))
        rows, fin = [], []
        for i in list(live):
            if i == 3 and step % 3 == 1:
                continue                                  # left out of this step, goes on later
            plan = plans.get(i, [])
            n = min(plan.pop(0) if plan else 1, len(reqs[i]) - at[i])
            rows.append((100 + i, reqs[i][at[i]:at[i] + n], list(range(n))))
            at[i] += n
            if at[i] == len(reqs[i]):
                fin.append(100 + i)
                live.remove(i)
        lg = eng.replay_step(rows, fin)
        k = 0
        for rid, t, _ in rows:
            got[rid - 100].append(lg[k:k + len(t)])
            k += len(t)
        step += 1
    for i in reqs:
        close(torch.cat(got[i]), want[i], dtype, f"request {i} in the batch")
    assert eng.sched.free_blocks() == 9 and eng.sched.free_state_slots() == 3


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_sizes_that_coincide_elsewhere(device, dtype):
    """One head everywhere, window 1 (a token sees itself only), a window longer than the
    sequence, kv_heads = heads, temperature steps of one token, diff 0, a rank larger than the
    width, layers without feed-forward first and last, width not a multiple of 8, a tight soft cap."""
    cd = cfg_dict([latent(heads=1, dim=4, vdim=12, kv_rank=50, window=1, ff=None),
                   attn(heads=1, kv_heads=1, dim=4, vdim=4, every=1, diff=0.0, coef=0.05),
                   hgrn(heads=1, dim=4, vdim=4), latent(heads=6, dim=12, vdim=4, kv_rank=8, window=1000),
                   attn(heads=6, kv_heads=6, dim=12, vdim=4, every=1000, ff=None)], width=36, vocab=61, cap=3.0,
                  scale=1.0)
    eng, cd, W = build(device, dtype, cd=cd)
    toks = tokens(140, vocab=61, seed=9)
    want = O.forward(cd, W, toks)
    close(replay_cuts(eng, toks, [66, 5]), want, dtype, "odd sizes")


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_long_decoding_through_windows_and_temperature_steps(device, dtype):
    """300 tokens decoded one by one after a short prompt: the latent window slides over decoded
    tokens only, the query temperature changes several times, the recurrent state is carried
    through hundreds of steps."""
    cd = cfg_dict([attn(every=64), latent(window=70), hgrn()])
    eng, cd, W = build(device, dtype, cd=cd)
    toks = tokens(330, seed=6)
    close(replay_cuts(eng, toks, [30]), O.forward(cd, W, toks), dtype, "long decoding")


@pytest.mark.parametrize("device,dtype", [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu)])
def test_greedy_generation_through_the_scheduler(device, dtype):
    """LLMEngine.generate: the engine's own scheduler chunks the prompts (a small token budget),
    batches the requests and decodes (hipGraph decode steps on the GPU); greedy tokens must
    equal the oracle's."""
    eng, cd, W = build(device, dtype, pages=16, max_batched_tokens=48, token_alignment=1, mixed_prefill_tokens=16)
    prompts = [tokens(90, seed=21), tokens(5, seed=22), tokens(67, seed=23)]
    reqs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    for p, r in zip(prompts, reqs):
        assert r.output_ids == O.greedy(cd, W, p, 12)
    assert eng.stats["prefill_steps"] > 2 and eng.sched.free_state_slots() == 4


@pytest.mark.parametrize("device", DEVICES)
def test_pipelined_generation_matches_synchronous(device):
    a, cd, W = build(device, "float32", async_decode=True)
    b, _, _ = build(device, "float32", async_decode=False)
    prompts = [tokens(40, seed=31), tokens(70, seed=32)]
    sp = SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True)
    assert [r.output_ids for r in a.generate(prompts, sp)] == [r.output_ids for r in b.generate(prompts, sp)]


@pytest.mark.parametrize("device", DEVICES)
def test_preemption_recomputes_state(device):
    """A pool too small for both sequences to grow: the scheduler preempts one (its pages and its
    state slot go back), recomputes it later from its first token, and the tokens do not change."""
    small, cd, W = build(device, "float32", pages=5)
    big, _, _ = build(device, "float32", pages=16)
    prompts = [tokens(120, seed=41), tokens(120, seed=42)]
    sp = SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True)
    got = [r.output_ids for r in small.generate(prompts, sp)]
    assert small.sched.preemptions() > 0
    assert got == [r.output_ids for r in big.generate(prompts, sp)]
    assert got[0] == O.greedy(cd, W, prompts[0], 20)
    assert small.sched.free_state_slots() == 4 and small.sched.free_blocks() == 5


def test_model_folder_roundtrip(tmp_path):
    """config.json + safetensors -> registry -> engine (EngineConfig.model as a folder)."""
    from nv_genai_amd.models.registry import read_config
    from nv_genai_amd.utils.checkpoint import save_weights

    cd = cfg_odd()
    cfg = BiruvikConfig.from_dict(cd)
    assert cfg.to_json_dict() == cd
    w = random_weights(cfg, 3, torch.bfloat16)
    save_weights(w, str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps(cd))
    got, cls = read_config(str(tmp_path))
    assert cls is BiruvikModel and got == cfg
    eng = LLMEngine(EngineConfig(model=str(tmp_path), dtype="float32", max_num_seqs=2, max_batched_tokens=128,
                                 max_model_len=128, kv_cache_blocks=4, detokenize=False, use_graphs=False,
                                 mixed_graphs=False, tuned_gemms=False, async_decode=False), device="cpu")
    toks = tokens(50, seed=7)
    close(eng.replay_step([(1, toks, list(range(50)))], [1]), O.forward(cd, w, toks), "float32", "model folder")
    sd = eng.model.state_dict()
    assert set(sd) == set(w)
    for k in w:
        assert torch.equal(sd[k].cpu().reshape(w[k].shape).to(w[k].dtype), w[k]), k


def test_config_errors():
    bad = cfg_odd()
    bad["layers"][0]["type"] = "conv"
    with pytest.raises(ValueError):
        BiruvikConfig.from_dict(bad)
    bad = cfg_dict([attn(heads=3, kv_heads=2)])
    with pytest.raises(ValueError):
        BiruvikConfig.from_dict(bad)
    cfg = BiruvikConfig.from_dict(cfg_odd())
    w = random_weights(cfg, 0)
    w["l0.mix.lower"] = w["l0.mix.lower"][:-1]
    with pytest.raises(ValueError):
        BiruvikModel(cfg, "cpu", torch.float32, weights=w)


def test_lambda_of_the_layer():
    cfg = BiruvikConfig.from_dict(cfg_dict([attn(dim=8, diff=0.2)]))
    w = random_weights(cfg, 4)
    m = BiruvikModel(cfg, "cpu", torch.float32, weights=w)
    f = {k: w["l0.mix." + k].double() for k in ("lq1", "lk1", "lq2", "lk2")}
    want = math.exp(float((f["lq1"] * f["lk1"]).sum())) - math.exp(float((f["lq2"] * f["lk2"]).sum())) + 0.2
    assert abs(m.layers[0]["lam"] - want) < 1e-12


@pytest.mark.gpu
def test_mfma_forms_run_and_agree_with_the_row_kernel():
    """bf16 rows with tile-sized heads take the MFMA kernels (not the row kernel); at sizes of real
    layers (long contexts, 128-wide heads, 16 heads per KV head, both maps, a window that starts
    and ends inside pages) the two forms agree to bf16 rounding."""
    torch.manual_seed(11)
    dev = "cuda"
    qa = torch.zeros(4, 256, dtype=torch.bfloat16, device=dev)
    assert ops.softmax_attention_mfma_ok(qa, 32, 64, 2, 2) and ops.softmax_attention_mfma_ok(qa, 256, 256, 16, 1)
    assert not ops.softmax_attention_mfma_ok(qa.float(), 32, 64, 2, 2)
    assert not ops.softmax_attention_mfma_ok(qa, 48, 64, 2, 2) and not ops.softmax_attention_mfma_ok(qa, 256, 64, 1, 2)
    for H, G, dk, dv, W, maps in ((8, 2, 128, 128, 0, 2), (16, 1, 128, 128, 300, 1), (4, 1, 256, 256, 1000, 1),
                                  (2, 2, 64, 128, 77, 2)):
        ctxs, qlens = [1500, 700, 65], [1500, 130, 1]
        nb, mb = 40, 24
        kc = (torch.randn(nb, G * maps, 64, dk, device=dev) * 0.5).bfloat16()
        vc = torch.randn(nb, G, 64, dv, device=dev).bfloat16()
        perm = torch.randperm(nb)[:36].tolist()
        bts = torch.zeros(3, mb, dtype=torch.int32)
        bts[0, :24] = torch.tensor(perm[:24])
        bts[1, :11] = torch.tensor(perm[24:35])
        bts[2, :2] = torch.tensor([perm[35], perm[0]])
        bts = bts.to(dev)
        T = sum(qlens)
        q = torch.randn(T, H * maps * dk, device=dev).bfloat16()
        gate = torch.randn(T, H, device=dev).bfloat16()
        cu = torch.tensor([0, 1500, 1630, 1631], dtype=torch.int32, device=dev)
        cx = torch.tensor(ctxs, dtype=torch.int32, device=dev)
        seq = torch.tensor([0] * 1500 + [1] * 130 + [2], dtype=torch.int32, device=dev)
        pos = torch.cat([torch.arange(c - n, c) for c, n in zip(ctxs, qlens)]).int().to(dev)
        kw = dict(window=W, maps=maps, lam=0.4, unit_eps=1e-5 if maps == 2 else None, out_scale=0.7, gate=gate)
        want = ops.softmax_attention(q, kc, vc, bts, seq, pos, H, G, dk, dv, dk ** -0.5, **kw).float()
        got = ops.softmax_attention_prefill(q, kc, vc, bts, cu, cx, 1500, H, G, dk, dv, dk ** -0.5, **kw).float()
        assert (got - want).abs().max().item() < 0.03 * max(1.0, want.abs().max().item()), ("prompt kernel", H, G, dk, dv, W)
        pick = torch.tensor([0, 63, 64, 700, 1499, 1500, 1629, 1630], device=dev)
        kw["gate"] = gate[pick].contiguous()
        got1 = ops.softmax_attention_rows(q[pick].contiguous(), kc, vc, bts, seq[pick].contiguous(),
                                          pos[pick].contiguous(), H, G, dk, dv, dk ** -0.5, max_ctx=1536, **kw).float()
        assert (got1 - want[pick]).abs().max().item() < 0.03 * max(1.0, want.abs().max().item()), ("single-token kernel", H, G, dk, dv, W)


@pytest.mark.parametrize("device", DEVICES)
def test_trace_runner_replays_a_schedule(device, tmp_path, monkeypatch, capsys):
    """The trace runner on a model folder: steps as JSON lines on standard input (a prompt in two
    portions, a second request beside single tokens of the first, requests ended and their names
    used again), logits files of the wanted places, a ``done`` line per step."""
    import io

    import numpy as np

    from nv_genai_amd.tools import trace_run
    from nv_genai_amd.utils.checkpoint import save_weights

    cd = cfg_dict([attn(), latent(window=9), hgrn()])
    cfg = BiruvikConfig.from_dict(cd)
    w = random_weights(cfg, 8, torch.bfloat16)
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    save_weights(w, str(model_dir))
    (model_dir / "config.json").write_text(json.dumps(cd))
    a, b = tokens(80, seed=51), tokens(30, seed=52)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:65], "want": [0, 64]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[65:78], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[:29], "want": [28]}, {"id": "a", "tokens": a[78:79], "want": [0]}],
              "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[79:], "want": [0]}, {"id": "b", "tokens": b[29:], "want": [0]}],
              "end": ["a", "b"]},
             {"step": 4, "entries": [{"id": "a", "tokens": b[:5], "want": [4]}], "end": ["a"]}]
    monkeypatch.setattr("sys.stdin", io.StringIO("".join(json.dumps(s) + "\n" for s in steps)))
    rc = trace_run.main(["--model", str(model_dir), "--dtype", "float32", "--out", str(out_dir), "--max-tokens", "192",
                         "--device", device])
    assert rc == 0
    assert [l for l in capsys.readouterr().out.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(5)]
    wa, wb = O.forward(cd, w, a), O.forward(cd, w, b)
    V = cd["vocab"]

    def rows(i):
        return torch.from_numpy(np.fromfile(out_dir / f"{i}.f32", dtype="<f4").reshape(-1, V).copy())

    assert not (out_dir / "1.f32").exists()
    close(rows(0), wa[[0, 64]], "float32", "first portion")
    close(rows(2), torch.stack([wb[28], wa[78]]), "float32", "a portion beside a single token")
    close(rows(3), torch.stack([wa[79], wb[29]]), "float32", "last tokens")
    close(rows(4), wb[4:5], "float32", "a name used again")
