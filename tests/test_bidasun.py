"""Bidasun on the serving engine against the plain oracle (tests/bidasun_oracle.py).

Every case runs twice: on the CPU (the engine on the fp32 reference ops: scheduling, pages,
state slots, row maps) and, marked ``gpu``, on the HIP kernels in float32 and bfloat16. The
models are small random ones built here; their sizes are chosen so that no two of heads,
kv heads, dim, vdim, window, keep_first and the page size coincide.
"""
import pytest
import torch

import bidasun_oracle as O
from nv_genai_amd import ops
from nv_genai_amd.engine.llm_engine import EngineConfig, LLMEngine, SamplingParams
from nv_genai_amd.models.bidasun import BidasunModel, random_weights
from nv_genai_amd.models.config import BidasunConfig

GPU = pytest.param("cuda", marks=pytest.mark.gpu)
DEVICES = ["cpu", GPU]


def cfg_dict(width=40, vocab=97, positions=512, layers=None, eps=1e-5):
    layers = layers or [
        dict(heads=4, kv_heads=2, dim=16, vdim=24, window=70, keep_first=3, scale=0.21, ff=56),
        dict(heads=3, kv_heads=3, dim=8, vdim=8, window=9, keep_first=0, scale=0.4, ff=None),
        dict(heads=2, kv_heads=1, dim=24, vdim=40, window=130, keep_first=66, scale=0.17, ff=72),
    ]
    return {"architecture": "Bidasun", "vocab": vocab, "width": width, "max_positions": positions,
            "norm": {"eps": eps},
            "layers": [{"type": "attention",
                        "mixer": {"heads": l["heads"], "kv_heads": l["kv_heads"], "dim": l["dim"], "vdim": l["vdim"],
                                  "scale": l["scale"], "mask": {"size": l["window"], "keep_first": l["keep_first"]}},
                        "mlp": None if l["ff"] is None else {"kind": "dense", "ff": l["ff"]}} for l in layers]}


def cfg_dict_tiles():
    """Head sizes the MFMA prompt kernel takes (32 / 64 / 128), unequal per block."""
    return cfg_dict(width=48, layers=[
        dict(heads=2, kv_heads=1, dim=32, vdim=64, window=70, keep_first=3, scale=0.2, ff=40),
        dict(heads=3, kv_heads=3, dim=64, vdim=32, window=9, keep_first=0, scale=0.15, ff=None),
        dict(heads=2, kv_heads=2, dim=128, vdim=128, window=130, keep_first=66, scale=0.1, ff=24)])


CFGS = {"odd": cfg_dict, "tiles": cfg_dict_tiles}


def build(device, dtype="float32", seed=0, pages=24, seqs=4, cd=None, graphs=None, **eng):
    cd = cd or cfg_dict()
    cfg = BidasunConfig.from_dict(cd)
    w = random_weights(cfg, seed, torch.bfloat16)       # bf16 values, as a checkpoint holds them
    tdt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    model = BidasunModel(cfg, device, tdt, weights=w)
    kw = dict(model="bidasun-test", dtype=dtype, max_num_seqs=seqs, max_batched_tokens=512,
              max_model_len=cfg.max_position, kv_cache_blocks=pages, detokenize=False,
              use_graphs=(device == "cuda") if graphs is None else graphs, graph_batch_sizes=(1, 2, 4),
              mixed_graphs=False, logits_tap=True, tuned_gemms=False, async_decode=False)
    kw.update(eng)
    e = LLMEngine(EngineConfig(**kw), device=device, model=model)
    return e, cd, {k: v.to(O.F64) for k, v in w.items()}


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


DTYPES = [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu),
          pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu)]


# ---------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("device", DEVICES)
def test_token_shift_and_state(device):
    torch.manual_seed(0)
    x = torch.randn(11, 20)
    mu = torch.rand(20)
    want = O.o_token_shift(x.double(), mu.double())
    # rows 0..4 in one step, 5..10 in the next: the second step reads row 4 from slot 2
    state = torch.zeros(3, 20, device=device)
    xd, mud = x.to(device), mu.to(device)
    src1 = torch.tensor([-1, 0, 1, 2, 3], dtype=torch.int32, device=device)
    h1 = ops.token_shift(xd[:5].contiguous(), mud, src1, state, torch.float32)
    ops.shift_save_(state, xd[:5].contiguous(), torch.tensor([4], dtype=torch.int32, device=device),
                    torch.tensor([2], dtype=torch.int32, device=device))
    src2 = torch.tensor([-4, 0, 1, 2, 3, 4], dtype=torch.int32, device=device)
    h2 = ops.token_shift(xd[5:].contiguous(), mud, src2, state, torch.float32)
    close(torch.cat([h1, h2]), want, "float32", "token shift")
    assert state[0].abs().sum() == 0 and state[1].abs().sum() == 0
    # decode rows: two sequences, one token each per step; the shift itself leaves x in the slots
    y = torch.randn(4, 2, 20)                            # [step, sequence, width]
    st = torch.zeros(3, 20, device=device)
    slots = torch.tensor([2, 0], dtype=torch.int32, device=device)
    outs = []
    for t in range(4):
        src = torch.tensor([-1, -1] if t == 0 else [-4, -2], dtype=torch.int32, device=device)
        outs.append(ops.token_shift(y[t].to(device).contiguous(), mud, src, st, torch.float32, save_slots=slots))
    for b in range(2):
        close(torch.stack([o[b] for o in outs]), O.o_token_shift(y[:, b].double(), mu.double()), "float32", "decode rows")
    assert st[1].abs().sum() == 0


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_postnorm_residual(device, dtype):
    torch.manual_seed(1)
    tdt = getattr(torch, dtype)
    x, y, w = torch.randn(7, 36), torch.randn(7, 36).to(tdt), torch.rand(36) + 0.5
    want = x.double() + O.o_rms(y.double(), w.double(), 1e-5)
    xd = x.to(device)
    cast = torch.empty(7, 36, dtype=tdt, device=device)
    ops.rmsnorm_residual_(xd, y.to(device), w.to(device), 1e-5, cast)
    close(xd, want, "float32", "residual")
    close(cast, want, dtype, "cast copy")
    rows = torch.tensor([6, 2], device=device)
    close(ops.rmsnorm_f32(xd, w.to(device), 1e-5, rows, tdt), O.o_rms(want[[6, 2]], w.double(), 1e-5), dtype, "last norm")


def _paged(q, k, v, device, tdt, bt_row):
    """Put k [T, G, dk], v [T, G, dv] into pages listed by bt_row; returns caches and slots."""
    T, G, dk = k.shape
    dv = v.shape[-1]
    nb = max(bt_row) + 1
    kc = torch.zeros(nb, G, 64, dk, dtype=tdt, device=device)
    vc = torch.zeros(nb, G, dv, 64, dtype=tdt, device=device)
    for t in range(T):
        kc[bt_row[t // 64], :, t % 64, :] = k[t].to(tdt).to(device)
        vc[bt_row[t // 64], :, :, t % 64] = v[t].to(tdt).to(device)
    return kc, vc


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_qk_norm_and_cache_write(device, dtype):
    torch.manual_seed(2)
    tdt = getattr(torch, dtype)
    # (heads, kv heads, dim, vdim, extra columns): unaligned rows, and 16-byte-aligned ones (vector kernel)
    for Hq, G, dk, dv, pad in ((4, 2, 8, 12, 5), (4, 2, 16, 8, 64), (40, 8, 128, 32, 0)):
        T = 70
        nq, nk, nv = Hq * dk, G * dk, G * dv
        proj = torch.randn(T, nq + nk + nv + pad).to(tdt)
        qw, kw = torch.rand(nq) + 0.5, torch.rand(nk) + 0.5
        bt = [5, 2]
        slots = torch.tensor([bt[t // 64] * 64 + t % 64 for t in range(T)], dtype=torch.int32)
        slots[3] = -1                                       # a row that writes nothing
        kc = torch.zeros(6, G, 64, dk, dtype=tdt, device=device)
        vc = torch.zeros(6, G, dv, 64, dtype=tdt, device=device)
        p64 = proj.double()
        pd = proj.clone().to(device)
        ops.qk_norm_cache_(pd, qw.to(device), kw.to(device), 1e-5, slots.to(device), kc, vc, Hq, G, dk, dv)
        close(pd[:, :nq], O.o_rms(p64[:, :nq], qw.double(), 1e-5), dtype, "q norm over the whole projection")
        kn = O.o_rms(p64[:, nq:nq + nk], kw.double(), 1e-5).view(T, G, dk)
        for t in (0, 63, 64, 69):
            close(kc[bt[t // 64], :, t % 64, :], kn[t], dtype, f"k page row {t}")
            close(vc[bt[t // 64], :, :, t % 64], p64[t, nq + nk:nq + nk + nv].view(G, dv), dtype, f"v page row {t}")
        assert kc[bt[0], :, 3].abs().sum() == 0
        close(pd[:, nq + nk:], p64[:, nq + nk:], dtype, "v and the rest untouched")


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_sigmoid_attention_random(device, dtype):
    torch.manual_seed(3)
    tdt = getattr(torch, dtype)
    for Hq, G, dk, dv, W, keep in ((4, 2, 16, 24, 70, 3), (3, 3, 8, 8, 9, 0), (2, 1, 24, 72, 130, 66), (1, 1, 4, 4, 1, 1)):
        T = 150
        q, k, v = torch.randn(T, Hq, dk).to(tdt), torch.randn(T, G, dk).to(tdt), torch.randn(T, G, dv).to(tdt)
        gate = torch.randn(T, Hq * dv).to(tdt)
        r1, r2, pb = torch.rand(Hq) + 0.5, torch.rand(Hq) * 0.5 + 0.05, torch.randn(Hq) - 1
        bt_row = [4, 0, 7]
        kc, vc = _paged(q, k, v, device, tdt, bt_row)
        bt = torch.tensor([[9, 9, 9], bt_row], dtype=torch.int32, device=device)
        want = O.o_sigmoid_attention(q.double(), k.double(), v.double(), Hq, G, 0.3, W, keep, r1.double(), r2.double(),
                                     pb.double()).reshape(T, -1) * torch.sigmoid(gate.double())
        pos = torch.arange(T, dtype=torch.int32, device=device)
        seq = torch.ones(T, dtype=torch.int32, device=device)
        got = ops.sigmoid_attention(q.reshape(T, -1).to(device), gate.to(device), kc, vc, bt, seq, pos, Hq, G, dk, dv,
                                    0.3, W, keep, r1.to(device), r2.to(device), pb.to(device))
        close(got, want, dtype, f"attention {Hq},{G},{dk},{dv},{W},{keep}")
        # the same rows one at a time, shuffled, as decode rows of a batch would come
        order = torch.randperm(T)[:40]
        got1 = ops.sigmoid_attention(q.reshape(T, -1)[order].contiguous().to(device), gate[order].contiguous().to(device),
                                     kc, vc, bt, seq[:40], pos[order.to(device)].contiguous(), Hq, G, dk, dv, 0.3, W,
                                     keep, r1.to(device), r2.to(device), pb.to(device))
        close(got1, want[order], dtype, "single rows")


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_one_key_stands_out(device, dtype):
    """Only one key scores high (q and that key scaled up, the rest pushed down by the per-head
    bias): the output is that key's value when the key is visible and zero when it is not. Run
    for keys far back, at page borders, at both edges of the window and of the kept prefix, as
    part of a prompt portion and as a single decode row."""
    tdt = getattr(torch, dtype)
    Hq = G = 1
    dk, dv, W, keep, T = 32, 32, 37, 5, 200
    r1, r2 = torch.tensor([0.0]), torch.tensor([0.3])
    pb = torch.tensor([-30.0])
    bt_row = [3, 1, 6, 2]
    bt = torch.tensor([bt_row], dtype=torch.int32, device=device)
    for i in (199, 128, 127, 64, 63, 40, 36, 5, 4, 0):
        cands = {0, keep - 1, keep, i - W, i - W + 1, i - 1, i, 63, 64, 127, 128, i // 2}
        for j in sorted(c for c in cands if 0 <= c <= i):
            k = torch.zeros(T, G, dk)
            k[j, 0, 0] = 8.0
            v = torch.randn(T, G, dv)
            q = torch.zeros(T, Hq, dk)
            q[:, 0, 0] = 8.0                              # q.k = 64 for key j, 0 for the rest
            kc, vc = _paged(q, k, v, device, tdt, bt_row)
            vis = O.o_visible(i, j, W, keep)
            want = v[j, 0].to(tdt).double() if vis else torch.zeros(dv, dtype=O.F64)
            for rows in (list(range(max(0, i - 2), i + 1)), [i]):     # a portion ending at i / i alone
                pos = torch.tensor(rows, dtype=torch.int32, device=device)
                seq = torch.zeros(len(rows), dtype=torch.int32, device=device)
                qr = q.reshape(T, -1)[rows].contiguous().to(tdt).to(device)
                tail = (Hq, G, dk, dv, 1.0, W, keep, r1.to(device), r2.to(device), pb.to(device))
                got = ops.sigmoid_attention(qr, None, kc, vc, bt, seq, pos, *tail)
                got3 = ops.sigmoid_attention_rows(qr, None, kc, vc, bt, seq, pos, *tail, max_ctx=256)
                err3 = (got3[-1].double().cpu() - want).abs().max().item()
                assert err3 < 1e-2, f"single-token kernel: query {i}, key {j}, visible {vis}: off by {err3}"
                if len(rows) > 1:   # the portion through the prompt kernel too (MFMA tiles in bf16 on the GPU)
                    cu = torch.tensor([0, len(rows)], dtype=torch.int32, device=device)
                    cx = torch.tensor([i + 1], dtype=torch.int32, device=device)
                    got2 = ops.sigmoid_attention_prefill(qr, None, kc, vc, bt, cu, cx, len(rows), *tail)
                    err2 = (got2[-1].double().cpu() - want).abs().max().item()
                    assert err2 < 1e-2, f"prompt kernel: query {i}, key {j}, visible {vis}: off by {err2}"
                err = (got[-1].double().cpu() - want).abs().max().item()
                assert err < 1e-2, f"query {i}, key {j}, visible {vis}: off by {err}"


@pytest.mark.parametrize("device,dtype", DTYPES)
def test_sigmoid_attention_prompt_portions(device, dtype):
    """The prompt-portion entry point (MFMA tiles for bf16 on the GPU): three sequences whose
    portions start in the middle of a page, end past a window and differ in length."""
    torch.manual_seed(4)
    tdt = getattr(torch, dtype)
    for Hq, G, dk, dv, W, keep in ((2, 1, 32, 64, 70, 3), (3, 3, 64, 32, 9, 0), (2, 2, 128, 128, 130, 66), (4, 2, 64, 64, 64, 64)):
        ctxs, qlens = [200, 67, 130], [150, 67, 2]
        r1, r2, pb = torch.rand(Hq) + 0.5, torch.rand(Hq) * 0.5 + 0.05, torch.randn(Hq) - 1
        bts = [[4, 0, 7, 9], [1, 2, 11, 11], [3, 5, 6, 11]]
        nb = 12
        kc = torch.zeros(nb, G, 64, dk, dtype=tdt, device=device)
        vc = torch.zeros(nb, G, dv, 64, dtype=tdt, device=device)
        qs, gs, wants = [], [], []
        for c, n, bt_row in zip(ctxs, qlens, bts):
            q, k, v = torch.randn(c, Hq, dk).to(tdt), torch.randn(c, G, dk).to(tdt), torch.randn(c, G, dv).to(tdt)
            gate = torch.randn(c, Hq * dv).to(tdt)
            for t in range(c):
                kc[bt_row[t // 64], :, t % 64, :] = k[t].to(device)
                vc[bt_row[t // 64], :, :, t % 64] = v[t].to(device)
            want = O.o_sigmoid_attention(q.double(), k.double(), v.double(), Hq, G, 0.2, W, keep, r1.double(),
                                         r2.double(), pb.double()).reshape(c, -1) * torch.sigmoid(gate.double())
            qs.append(q.reshape(c, -1)[c - n:])
            gs.append(gate[c - n:])
            wants.append(want[c - n:])
        cu = torch.tensor([0, 150, 217, 219], dtype=torch.int32, device=device)
        got = ops.sigmoid_attention_prefill(torch.cat(qs).to(device), torch.cat(gs).to(device), kc, vc,
                                            torch.tensor(bts, dtype=torch.int32, device=device), cu,
                                            torch.tensor(ctxs, dtype=torch.int32, device=device), 150, Hq, G, dk, dv,
                                            0.2, W, keep, r1.to(device), r2.to(device), pb.to(device))
        close(got, torch.cat(wants), dtype, f"prompt portions {Hq},{G},{dk},{dv},{W},{keep}")
        # the same rows as single-token rows of a batch (page-parallel MFMA kernel for bf16 on the GPU)
        seq = torch.tensor([0] * 150 + [1] * 67 + [2] * 2, dtype=torch.int32, device=device)
        pos = torch.cat([torch.arange(c - n, c) for c, n in zip(ctxs, qlens)]).int().to(device)
        pick = torch.tensor([0, 13, 149, 150, 216, 217, 218, 77], device=device)
        got1 = ops.sigmoid_attention_rows(torch.cat(qs).to(device)[pick].contiguous(), torch.cat(gs).to(device)[pick].contiguous(),
                                          kc, vc, torch.tensor(bts, dtype=torch.int32, device=device),
                                          seq[pick].contiguous(), pos[pick].contiguous(), Hq, G, dk, dv, 0.2, W, keep,
                                          r1.to(device), r2.to(device), pb.to(device), max_ctx=256)
        close(got1, torch.cat(wants)[pick.cpu()], dtype, "single-token rows")


# ---------------------------------------------------------------------------- the model on the engine
@pytest.mark.parametrize("shape", sorted(CFGS))
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_whole_prompt_and_layers(device, dtype, shape):
    eng, cd, W = build(device, dtype, cd=CFGS[shape]())
    toks = tokens(200)
    want, layers = O.o_forward(cd, W, toks)
    tap = []
    got = eng.replay_step([(1, toks, list(range(len(toks))))], [1], layer_tap=tap)
    for i, (a, b) in enumerate(zip(tap, layers)):
        close(a, b, dtype, f"residual stream after block {i}")
    close(got, want, dtype, "logits")
    # the very first tokens: nothing before them, a shift from zeros
    close(got[:3], O.o_forward(cd, W, toks[:3])[0], dtype, "first tokens")


@pytest.mark.parametrize("shape", sorted(CFGS))
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_prefill_then_decode_and_portions(device, dtype, shape):
    eng, cd, W = build(device, dtype, cd=CFGS[shape]())
    toks = tokens(230, seed=5)
    want = O.o_forward(cd, W, toks)[0]
    close(replay_cuts(eng, toks, [70]), want, dtype, "prompt then token by token (160 decoded, windows pass)")
    close(replay_cuts(eng, toks, [1] * 3 + [2, 61, 2, 3, 64, 2, 63, 2, 17]), want, dtype, "portions down to two tokens")
    close(replay_cuts(eng, toks, []), want, dtype, "token by token from the first")
    assert eng.sched.free_blocks() == eng.num_blocks and eng.sched.free_state_slots() == 4


@pytest.mark.parametrize("shape", sorted(CFGS))
@pytest.mark.parametrize("device,dtype", DTYPES)
def test_mixed_batches_and_reuse(device, dtype, shape):
    """Four unequal requests interleaved (portions beside single tokens, a request that skips
    steps), in a pool that only holds the live ones: pages and slots are freed and used again by
    requests that start later. Every request must equal its run alone (the oracle)."""
    eng, cd, W = build(device, dtype, pages=9, seqs=3, cd=CFGS[shape]())
    reqs = {i: tokens(n, seed=10 + i) for i, n in enumerate((150, 65, 1, 200, 129, 64, 3))}
    want = {i: O.o_forward(cd, W, t)[0] for i, t in reqs.items()}
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
    """One head, one kv head, window 1 (a token sees itself and the kept ones), keep_first past a
    page, vdim != dim, a block without feed-forward first, width not a multiple of 8."""
    cd = cfg_dict(width=36, vocab=61, layers=[
        dict(heads=1, kv_heads=1, dim=4, vdim=12, window=1, keep_first=70, scale=1.0, ff=None),
        dict(heads=6, kv_heads=2, dim=12, vdim=4, window=64, keep_first=1, scale=0.05, ff=20)])
    eng, cd, W = build(device, dtype, cd=cd)
    toks = tokens(140, vocab=61, seed=9)
    want = O.o_forward(cd, W, toks)[0]
    close(replay_cuts(eng, toks, [66, 5]), want, dtype, "odd sizes")


@pytest.mark.parametrize("device,dtype", [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu)])
def test_greedy_generation_through_the_scheduler(device, dtype):
    """LLMEngine.generate: the engine's own scheduler chunks the prompts (a small token budget),
    batches the requests and decodes (hipGraph decode steps on the GPU); greedy tokens must
    equal the oracle's."""
    eng, cd, W = build(device, dtype, pages=16, max_batched_tokens=48, token_alignment=1, mixed_prefill_tokens=16)
    prompts = [tokens(90, seed=21), tokens(5, seed=22), tokens(67, seed=23)]
    reqs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    for p, r in zip(prompts, reqs):
        assert r.output_ids == O.o_greedy(cd, W, p, 12)
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
    assert got[0] == O.o_greedy(cd, W, prompts[0], 20)
    assert small.sched.free_state_slots() == 4 and small.sched.free_blocks() == 5


def test_model_folder_roundtrip(tmp_path):
    """config.json + safetensors -> registry -> engine (EngineConfig.model as a folder)."""
    import json

    from nv_genai_amd.models.registry import read_config
    from nv_genai_amd.utils.checkpoint import save_weights

    cd = cfg_dict()
    cfg = BidasunConfig.from_dict(cd)
    assert cfg.to_json_dict() == cd
    w = random_weights(cfg, 3, torch.bfloat16)
    save_weights(w, str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps(cd))
    got_cfg, cls = read_config(str(tmp_path))
    assert cls is BidasunModel and got_cfg == cfg
    eng = LLMEngine(EngineConfig(model=str(tmp_path), dtype="float32", max_num_seqs=2, max_batched_tokens=128,
                                 max_model_len=256, kv_cache_blocks=8, detokenize=False, use_graphs=False,
                                 tuned_gemms=False), device="cpu")
    toks = tokens(30)
    want = O.o_forward(cd, {k: v.to(O.F64) for k, v in w.items()}, toks)[0]
    close(eng.replay_step([(1, toks, [29])], [1]), want[29:], "float32", "folder model")


def test_scheduler_state_slots():
    from nv_genai_amd._native import rt

    s = rt.Scheduler(8, 64, 2, 256, 512, False)
    s.set_state_slots(2)
    s.add(1, [1, 2, 3], 0)
    s.add(2, [4] * 70, 0)
    import numpy as np

    bufs = [np.zeros(256, np.int32) for _ in range(3)] + [np.zeros(3, np.int32), np.zeros(2, np.int32),
                                                         np.zeros((2, 8), np.int32), np.zeros(2, np.int64),
                                                         np.zeros(2, np.int32)]
    kind, n, ntok = s.schedule_rows([1, 2], [3, 64], *bufs)
    assert (kind, n, ntok) == (1, 2, 67) and {s.state_slot(1), s.state_slot(2)} == {0, 1}
    kind, n, ntok = s.schedule_rows([2], [1], *bufs)       # a single continuation token: a decode row
    assert (kind, n, ntok) == (2, 1, 1) and bufs[1][0] == 64 and s.used_blocks() == 3
    with pytest.raises(RuntimeError):
        s.schedule_rows([1], [1], *bufs)                   # no tokens left
    s.extend(1, [9, 9])
    kind, n, ntok = s.schedule_rows([2, 1], [5, 2], *bufs)
    assert kind == 1 and list(bufs[6][:2]) == [2, 1] and list(bufs[1][:7]) == [65, 66, 67, 68, 69, 3, 4]
    s.finish(1)
    assert s.free_state_slots() == 1
    s.add(3, [5], 0)
    s.schedule_rows([3], [1], *bufs)
    assert s.state_slot(3) == 0 or s.state_slot(3) == 1
    s.add(4, [5], 0)
    with pytest.raises(RuntimeError):
        s.schedule_rows([4], [1], *bufs)                   # both slots taken
