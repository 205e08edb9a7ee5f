"""Biruvik decoder on the gfx950 kernel set: sandwich-normed sub-layers on an fp32 residual
stream, three kinds of mixer chosen per layer, relu^2 feed-forward, soft-capped logits.

Per layer (``x`` is the fp32 residual stream, activations in the model dtype; every norm is an
RMS norm with a single gain):

    h  = norm1(x)                       fused into the previous residual step
    x += norm1b(mixer(h)); h2 = norm2(x)            ops.rmsnorm_residual_next_
    x += norm2b(down(relu(up h2)^2)); h = next layer's norm1(x)      (same op)

Mixers:

* ``attention`` — differential softmax attention. One GEMM gives q | k | v; ``ops.headnorm_cache_``
  adds the biases, RMS-normalises every (head, map) of q and k, applies the query temperature and
  writes the pages; ``ops.softmax_attention`` runs both maps of a head, combines them as
  ``a1 - lam * a2`` and brings the head to unit RMS.
* ``latent_attention`` — only the normalised latent c [kv_rank] of a token is cached. The key
  expansion is folded into the query (``(W_uk c) . q = c . (W_uk^T q)``) and the value expansion is
  applied to the attention output, so the attention itself is multi-query attention whose keys and
  values are both the latent page (window, per-head sigmoid gate in the same kernel).
* ``hgrn2`` — ``ops.hgrn2_scan`` carries the fp32 state [heads, dim, vdim] of every sequence in a
  state slot handed out by the scheduler; ``ops.group_rmsnorm`` normalises the heads.

The serving engine drives this class as it drives the other decoders (``forward`` on a step's token
rows + ``logits``); ``AttnMeta`` carries the per-step row maps (``tok_seq``, ``state_slots``).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from .. import ops
from ..parallel.dist import ParallelContext, get_context
from .config import BiruvikConfig
from .llama import AttnMeta


def _ceil8(n: int) -> int:
    return (n + 7) // 8 * 8


class BiruvikModel:
    stateful = True                # recurrent layers keep per-sequence state in scheduler slots
    uses_decode_workspace = False
    supports_step_graphs = False   # prefill / mixed steps run eagerly (decode steps are graphs)
    supports_prefix_cache = False  # a cached page carries no recurrent state

    def __init__(self, cfg: BiruvikConfig, device="cuda", dtype=torch.bfloat16,
                 pctx: Optional[ParallelContext] = None, seed: int = 0,
                 weights: Optional[Dict[str, torch.Tensor]] = None, fp8: bool = False):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Biruvik runs in bfloat16 or float32")
        if fp8:
            raise NotImplementedError("FP8 projections cover the Llama-layout decoders")
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.p = pctx or get_context()
        if self.p.tp_size > 1 or self.p.pp_size > 1:
            raise NotImplementedError("Biruvik runs on one GPU per replica (no TP / PP split)")
        self.fp8 = False
        self.kv_dtype, self.kv_scales = "auto", (1.0, 1.0)
        self.sequence_parallel, self.sp_min_tokens, self.split_mixed, self.moe_ws = False, 0, False, None
        m0 = cfg.blocks[0].mixer
        self.hq, self.hkv, self.D = m0.heads, getattr(m0, "kv_heads", 1), m0.dim
        self.vocab_local = cfg.vocab_size
        self.k_cache: List[Optional[torch.Tensor]] = []
        self.v_cache: List[Optional[torch.Tensor]] = []
        self.rec_state: List[Optional[torch.Tensor]] = []
        self.skinny = (self.device.type == "cuda" and dtype == torch.bfloat16 and ops.skinny.enabled())
        self.mfma = True   # MFMA attention kernels where they apply (bf16, tile-sized heads)
        if weights is None:
            weights = random_weights(cfg, seed, dtype)
        self._load(weights)

    # ------------------------------------------------------------------ weights
    def _load(self, w: Dict[str, torch.Tensor]):
        cfg, dev, dt = self.cfg, self.device, self.dtype
        H = cfg.hidden

        def mat(name, shape):
            t = w[name]
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(t.shape)}, config says {tuple(shape)}")
            t = t.to(dev, dt).contiguous()
            return t.clone() if t.data_ptr() % 16 else t   # (a memory-mapped file need not be aligned)

        def vec(name, n):
            t = w[name].to(dev, torch.float32).reshape(-1).contiguous()
            if t.numel() != n:
                raise ValueError(f"{name}: {t.numel()} elements, config says {n}")
            return t

        def fused(*mats):
            """Row-stacked GEMM weight, padded with zero rows to a multiple of 8 outputs."""
            W = torch.cat(mats)
            pad = _ceil8(W.shape[0]) - W.shape[0]
            if pad:
                W = torch.cat([W, torch.zeros(pad, W.shape[1], dtype=W.dtype, device=W.device)])
            return W.contiguous()

        self.embed = mat("embed", (cfg.vocab_size, H))
        self.layers: List[dict] = []
        for i, b in enumerate(cfg.blocks):
            p, m = f"l{i}.", b.mixer
            L = {"type": b.type, "spec": m, "norm1": vec(p + "norm1", 1), "norm1b": vec(p + "norm1b", 1)}
            if b.type == "attention":
                nq, nk, nv = 2 * m.heads * m.dim, 2 * m.kv_heads * m.dim, m.kv_heads * m.vdim
                L["wqkv"] = fused(mat(p + "mix.q", (nq, H)), mat(p + "mix.k", (nk, H)), mat(p + "mix.v", (nv, H)))
                L["bias"] = torch.cat([vec(p + "mix.q.b", nq), vec(p + "mix.k.b", nk), vec(p + "mix.v.b", nv)])
                L["qn"], L["kn"] = vec(p + "mix.q.norm", m.dim), vec(p + "mix.k.norm", m.dim)
                lv = {k: w[p + "mix." + k].double().reshape(-1) for k in ("lq1", "lk1", "lq2", "lk2")}
                if any(t.numel() != m.dim for t in lv.values()):
                    raise ValueError(f"layer {i}: lambda vectors do not fit the config")
                L["lam_vec"] = {k: t.float() for k, t in lv.items()}
                L["lam"] = (math.exp(float((lv["lq1"] * lv["lk1"]).sum()))
                            - math.exp(float((lv["lq2"] * lv["lk2"]).sum())) + m.diff)
                L["wo"] = mat(p + "mix.o", (H, m.heads * m.vdim))
            elif b.type == "latent_attention":
                nq, r = m.heads * m.dim, m.kv_rank
                L["wqcg"] = fused(mat(p + "mix.q", (nq, H)), mat(p + "mix.dkv", (r, H)), mat(p + "mix.g", (m.heads, H)))
                L["cn"] = vec(p + "mix.dkv.norm", r)
                # per head: W_uk [dim, r] folds into the query, W_uv^T [r, vdim] expands the output
                L["wuk"] = mat(p + "mix.uk", (nq, r)).view(m.heads, m.dim, r).contiguous()
                L["wuvT"] = mat(p + "mix.uv", (m.heads * m.vdim, r)).view(m.heads, m.vdim, r).transpose(1, 2).contiguous()
                L["wo"] = mat(p + "mix.o", (H, m.heads * m.vdim))
            elif b.type == "hgrn2":
                nq, nv = m.heads * m.dim, m.heads * m.vdim
                L["wqfv"] = fused(mat(p + "mix.q", (nq, H)), mat(p + "mix.f", (nq, H)), mat(p + "mix.v", (nv, H)))
                L["fb"], L["lower"] = vec(p + "mix.f.b", nq), vec(p + "mix.lower", nq)
                L["on"] = vec(p + "mix.norm", m.vdim)
                L["wo"] = mat(p + "mix.o", (H, nv))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {b.type!r}")
            if b.mlp is not None:
                L["wu"], L["wd"] = mat(p + "mlp.up", (b.mlp.ff, H)), mat(p + "mlp.down", (H, b.mlp.ff))
                L["norm2"], L["norm2b"] = vec(p + "norm2", 1), vec(p + "norm2b", 1)
            self.layers.append(L)
        self.final_norm = vec("final.norm", 1)
        # the row-gather norm kernels take a weight per coordinate
        self._first_norm = self.layers[0]["norm1"].expand(H).contiguous()
        self._final_norm = self.final_norm.expand(H).contiguous()
        last = self.layers[-1]
        self._last_post = (last["norm2b"] if "wu" in last else last["norm1b"]).expand(H).contiguous()
        self.lm_head = mat("head", (cfg.vocab_size, H))

    def state_dict(self) -> Dict[str, torch.Tensor]:
        dt = self.dtype
        out = {"embed": self.embed, "final.norm": self.final_norm.reshape(()).to(dt), "head": self.lm_head}
        for i, L in enumerate(self.layers):
            p, m = f"l{i}.", L["spec"]
            for k in ("norm1", "norm1b", "norm2", "norm2b"):
                if k in L:
                    out[p + k] = L[k].reshape(()).to(dt)
            out[p + "mix.o"] = L["wo"]
            if L["type"] == "attention":
                nq, nk, nv = 2 * m.heads * m.dim, 2 * m.kv_heads * m.dim, m.kv_heads * m.vdim
                W, B = L["wqkv"], L["bias"].to(dt)
                out.update({p + "mix.q": W[:nq], p + "mix.k": W[nq:nq + nk], p + "mix.v": W[nq + nk:nq + nk + nv],
                            p + "mix.q.b": B[:nq], p + "mix.k.b": B[nq:nq + nk], p + "mix.v.b": B[nq + nk:],
                            p + "mix.q.norm": L["qn"].to(dt), p + "mix.k.norm": L["kn"].to(dt)})
                out.update({p + "mix." + k: t.to(dt) for k, t in L["lam_vec"].items()})
            elif L["type"] == "latent_attention":
                nq, r = m.heads * m.dim, m.kv_rank
                W = L["wqcg"]
                out.update({p + "mix.q": W[:nq], p + "mix.dkv": W[nq:nq + r], p + "mix.g": W[nq + r:nq + r + m.heads],
                            p + "mix.dkv.norm": L["cn"].to(dt), p + "mix.uk": L["wuk"].reshape(nq, r),
                            p + "mix.uv": L["wuvT"].transpose(1, 2).reshape(m.heads * m.vdim, r)})
            else:
                nq, nv = m.heads * m.dim, m.heads * m.vdim
                W = L["wqfv"]
                out.update({p + "mix.q": W[:nq], p + "mix.f": W[nq:2 * nq], p + "mix.v": W[2 * nq:2 * nq + nv],
                            p + "mix.f.b": L["fb"].to(dt), p + "mix.lower": L["lower"].to(dt),
                            p + "mix.norm": L["on"].to(dt)})
            if "wu" in L:
                out.update({p + "mlp.up": L["wu"], p + "mlp.down": L["wd"]})
        return out

    # ------------------------------------------------------------------ cache and state
    def allocate_kv_cache(self, num_blocks: int, block_size: int = 64, kv_dtype: str = "auto",
                          kv_scales=(1.0, 1.0)):
        """Row-major pages in the model dtype, all layers addressed by the same page numbers:
        ``attention`` layers K [blocks, 2 * kv_heads, 64, dim] (both maps) and V [blocks,
        kv_heads, 64, vdim]; ``latent_attention`` layers one latent page [blocks, 1, 64, kv_rank]
        that serves as keys and values; ``hgrn2`` layers none."""
        if block_size != 64:
            raise ValueError("the gfx950 attention kernels use 64-token KV pages")
        if kv_dtype not in ("auto", "bf16"):
            raise ValueError("Biruvik keeps its KV pages in the model dtype")
        self.k_cache, self.v_cache = [], []

        def pages(heads, d):
            return torch.zeros(num_blocks, heads, block_size, d, device=self.device, dtype=self.dtype)

        for L in self.layers:
            m = L["spec"]
            if L["type"] == "attention":
                self.k_cache.append(pages(2 * m.kv_heads, m.dim))
                self.v_cache.append(pages(m.kv_heads, m.vdim))
            elif L["type"] == "latent_attention":
                c = pages(1, m.kv_rank)
                self.k_cache.append(c)
                self.v_cache.append(c)
            else:
                self.k_cache.append(None)
                self.v_cache.append(None)
        return self.k_cache, self.v_cache

    def allocate_state(self, slots: int) -> None:
        """Recurrent state: per ``hgrn2`` layer fp32 [slots, heads, dim, vdim]. A slot needs no
        clearing when it is given to a new sequence: a segment that starts at position 0 starts
        from zeros, not from the slot."""
        self.rec_state = [torch.zeros(max(1, slots), L["spec"].heads, L["spec"].dim, L["spec"].vdim,
                                      device=self.device, dtype=torch.float32) if L["type"] == "hgrn2" else None
                          for L in self.layers]

    def kv_block_bytes(self, block_size: int = 64, kv_dtype: str = "auto") -> int:
        elem = torch.finfo(self.dtype).bits // 8
        n = 0
        for b in self.cfg.blocks:
            m = b.mixer
            if b.type == "attention":
                n += m.kv_heads * (2 * m.dim + m.vdim)
            elif b.type == "latent_attention":
                n += m.kv_rank
        return max(1, n) * block_size * elem

    def copy_kv_blocks(self, src, dst) -> None:
        raise NotImplementedError("beam search forks need a copy of the recurrent state")

    def ipc_collectives_cover(self, rows: int, tokens: int) -> bool:
        return True

    def quantize_fp8(self) -> None:
        raise NotImplementedError("FP8 projections cover the Llama-layout decoders")

    # ------------------------------------------------------------------ forward
    def _lin(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """x @ w^T: decode-shape rows take the skinny MFMA GEMM where the measured table
        (ops.skinny) holds this (N, K) and prefers it over the library GEMM."""
        if self.skinny and x.shape[0] <= 512 and x.stride(1) == 1 and x.stride(0) % 8 == 0:
            pk = ops.skinny.table().pick(w.shape[0], w.shape[1], x.shape[0])
            if pk is not None:
                cfg, split = pk
                if split == 1:
                    return ops.skinny_gemm(x, w, cfg, 1, 0)
                return ops.PartialSum(ops.skinny_gemm(x, w, cfg, split, 1)).materialize()
        return ops.linear(x, w)

    def _attend(self, q, gate, kc, vc, pos, meta: AttnMeta, H, G, dk, dv, **kw):
        """Softmax attention of a step's rows: prompt portions on the MFMA tile kernel and
        single-token rows on the page-parallel kernel where they apply (bf16, tile-sized
        heads), everything else on the row kernel."""
        if self.mfma and ops.softmax_attention_mfma_ok(q, dk, dv, H // G, kw.get("maps", 1)):
            nd = meta.n_decode if meta.kind == "mixed" else (q.shape[0] if meta.kind == "decode" else 0)
            out = torch.empty(q.shape[0], H * dv, dtype=q.dtype, device=q.device)
            if nd:
                ops.softmax_attention_rows(q[:nd], kc, vc, meta.block_tables, meta.tok_seq[:nd], pos[:nd], H, G, dk,
                                           dv, max_ctx=meta.max_ctx, gate=None if gate is None else gate[:nd],
                                           out=out[:nd], **kw)
            if nd < q.shape[0]:
                ops.softmax_attention_prefill(q[nd:], kc, vc, meta.block_tables[nd:],
                                              meta.cu_q_prefill if nd else meta.cu_q, meta.ctx_lens[nd:],
                                              meta.max_q_len, H, G, dk, dv,
                                              gate=None if gate is None else gate[nd:], out=out[nd:], **kw)
            return out
        return ops.softmax_attention(q, kc, vc, meta.block_tables, meta.tok_seq, pos, H, G, dk, dv, gate=gate, **kw)

    def _mix_attention(self, li: int, h, pos, meta: AttnMeta):
        L = self.layers[li]
        m = L["spec"]
        nq = 2 * m.heads * m.dim
        proj = self._lin(h, L["wqkv"])
        ops.headnorm_cache_(proj, meta.slots, self.k_cache[li], self.v_cache[li], 2 * m.heads, 2 * m.kv_heads, m.dim,
                            m.kv_heads, m.vdim, self.cfg.eps, q_w=L["qn"], k_w=L["kn"], bias=L["bias"], pos=pos,
                            temp_coef=m.q_temp_coef, temp_every=m.q_temp_every)
        a = self._attend(proj[:, :nq], None, self.k_cache[li], self.v_cache[li], pos, meta, m.heads, m.kv_heads,
                         m.dim, m.vdim, scale=m.scale, window=0, maps=2, lam=L["lam"], unit_eps=self.cfg.eps,
                         out_scale=1.0 - m.diff)
        return self._lin(a, L["wo"])

    def _mix_latent(self, li: int, h, pos, meta: AttnMeta):
        L = self.layers[li]
        m = L["spec"]
        T, nq, r = h.shape[0], m.heads * m.dim, m.kv_rank
        proj = self._lin(h, L["wqcg"])
        cc = self.k_cache[li]
        ops.headnorm_cache_(proj[:, nq:], meta.slots, cc, None, 0, 1, r, 0, 0, self.cfg.eps, k_w=L["cn"])
        q = proj[:, :nq].view(T, m.heads, m.dim).transpose(0, 1)             # [H, T, dim] view
        ql = torch.bmm(q, L["wuk"]).transpose(0, 1).reshape(T, m.heads * r)  # rows [H * r]
        gate = proj[:, nq + r:nq + r + m.heads]
        a = self._attend(ql, gate, cc, cc, pos, meta, m.heads, 1, r, r, scale=m.scale, window=m.window)
        av = torch.bmm(a.view(T, m.heads, r).transpose(0, 1), L["wuvT"])     # [H, T, vdim]
        return self._lin(av.transpose(0, 1).reshape(T, m.heads * m.vdim), L["wo"])

    def _mix_hgrn2(self, li: int, h, pos, meta: AttnMeta):
        L = self.layers[li]
        m = L["spec"]
        proj = self._lin(h, L["wqfv"])
        o = ops.hgrn2_scan(proj, L["fb"], L["lower"], self.rec_state[li], m.heads, m.dim, m.vdim,
                           None if meta.kind == "decode" else meta.cu_q, meta.state_slots, pos)
        return self._lin(ops.group_rmsnorm(o, L["on"], m.heads, self.cfg.eps, self.dtype), L["wo"])

    def forward(self, ids: torch.Tensor, pos: torch.Tensor, meta: AttnMeta,
                sample_idx: Optional[torch.Tensor] = None, embed_override=None,
                layer_tap: Optional[list] = None) -> torch.Tensor:
        """Final-normed rows selected by ``sample_idx`` (all rows if None) of a step's token rows.
        ``layer_tap``: a list that receives a copy of the residual stream after every layer."""
        if embed_override is not None:
            raise NotImplementedError("Biruvik takes token ids only")
        if meta.tok_seq is None or meta.state_slots is None:
            raise ValueError("Biruvik steps need the engine's row maps (tok_seq, state slots)")
        eps, dt = self.cfg.eps, self.dtype
        x = ops.embed_rows(ids, self.embed, self.cfg.embed_scale)
        h = ops.rmsnorm_f32(x, self._first_norm, eps, dtype=dt)
        mixers = {"attention": self._mix_attention, "latent_attention": self._mix_latent, "hgrn2": self._mix_hgrn2}
        n = len(self.layers)
        for li, L in enumerate(self.layers):
            y, post = mixers[L["type"]](li, h, pos, meta), L["norm1b"]
            if "wu" in L:
                h2 = ops.rmsnorm_residual_next_(x, y, post, eps, L["norm2"], dt)
                y, post = self._lin(ops.relu_sq(self._lin(h2, L["wu"])), L["wd"]), L["norm2b"]
            if li + 1 < n:
                h = ops.rmsnorm_residual_next_(x, y, post, eps, self.layers[li + 1]["norm1"], dt)
            else:
                ops.rmsnorm_residual_(x, y, self._last_post, eps)
            if layer_tap is not None:
                layer_tap.append(x.clone())
        return ops.rmsnorm_f32(x, self._final_norm, eps, rows=sample_idx, dtype=dt)

    def logits(self, h: torch.Tensor) -> torch.Tensor:
        z = ops.linear(h, self.lm_head).float()
        if self.cfg.logit_softcap > 0:
            ops.softcap_(z, self.cfg.logit_softcap)
        return z


def random_weights(cfg: BiruvikConfig, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random weights under the checkpoint's tensor names (benchmarks, tests, smoke runs)."""
    g = torch.Generator().manual_seed(seed)
    H = cfg.hidden

    def rnd(*shape, std):
        return (torch.randn(*shape, generator=g) * std).to(dtype)

    def gain(lo=0.6, hi=1.4):
        return (lo + (hi - lo) * torch.rand((), generator=g)).to(dtype)

    def around1(n):
        return (1.0 + 0.1 * torch.randn(n, generator=g)).to(dtype)

    w = {"embed": rnd(cfg.vocab_size, H, std=1.0), "final.norm": gain(), "head": rnd(cfg.vocab_size, H, std=H ** -0.5)}
    s = H ** -0.5
    for i, b in enumerate(cfg.blocks):
        p, m = f"l{i}.", b.mixer
        w.update({p + "norm1": gain(), p + "norm1b": gain(0.3, 0.8)})
        if b.type == "attention":
            nq, nk, nv = 2 * m.heads * m.dim, 2 * m.kv_heads * m.dim, m.kv_heads * m.vdim
            w.update({p + "mix.q": rnd(nq, H, std=s), p + "mix.k": rnd(nk, H, std=s), p + "mix.v": rnd(nv, H, std=s),
                      p + "mix.q.b": rnd(nq, std=0.1), p + "mix.k.b": rnd(nk, std=0.1), p + "mix.v.b": rnd(nv, std=0.1),
                      p + "mix.q.norm": around1(m.dim), p + "mix.k.norm": around1(m.dim),
                      p + "mix.o": rnd(H, m.heads * m.vdim, std=(m.heads * m.vdim) ** -0.5)})
            for k in ("lq1", "lk1", "lq2", "lk2"):
                w[p + "mix." + k] = rnd(m.dim, std=0.1)
        elif b.type == "latent_attention":
            nq, r = m.heads * m.dim, m.kv_rank
            w.update({p + "mix.q": rnd(nq, H, std=s), p + "mix.dkv": rnd(r, H, std=s), p + "mix.dkv.norm": around1(r),
                      p + "mix.uk": rnd(nq, r, std=r ** -0.5), p + "mix.uv": rnd(m.heads * m.vdim, r, std=r ** -0.5),
                      p + "mix.g": rnd(m.heads, H, std=s),
                      p + "mix.o": rnd(H, m.heads * m.vdim, std=(m.heads * m.vdim) ** -0.5)})
        else:
            nq, nv = m.heads * m.dim, m.heads * m.vdim
            w.update({p + "mix.q": rnd(nq, H, std=s), p + "mix.f": rnd(nq, H, std=s), p + "mix.v": rnd(nv, H, std=s),
                      p + "mix.f.b": rnd(nq, std=0.5), p + "mix.lower": (0.9 * torch.rand(nq, generator=g)).to(dtype),
                      p + "mix.norm": around1(m.vdim), p + "mix.o": rnd(H, nv, std=nv ** -0.5)})
        if b.mlp is not None:
            F = b.mlp.ff
            w.update({p + "mlp.up": rnd(F, H, std=s), p + "mlp.down": rnd(H, F, std=F ** -0.5),
                      p + "norm2": gain(), p + "norm2b": gain(0.3, 0.8)})
    return w
