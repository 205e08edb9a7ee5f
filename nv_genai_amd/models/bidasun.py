"""Bidasun decoder on the gfx950 kernel set: post-norm blocks on an fp32 residual stream,
learned positions, token shift in front of every mixer, gated sigmoid attention.

Per block (``x`` is the fp32 residual stream, activations in the model dtype):

    h    = x + (x_prev - x) * shift                  ops.token_shift   (x_prev: previous token's x)
    proj = h @ [Wq | Wk | Wv | Wg]^T                 one library GEMM
    q, k = rmsnorm over the whole projection; K / V^T page write      ops.qk_norm_cache_
    a    = sum_j sigmoid(q.k_j s - r1 ln(1 + r2 (i - j)) + pb) v_j    ops.sigmoid_attention
           over j <= i with (i - j < window or j < keep_first), times sigmoid(g)
    x   += rmsnorm(a @ Wo^T) * w1                    ops.rmsnorm_residual_ (+ bf16 copy of x)
    x   += rmsnorm(down(gelu_tanh(gate x) * up x)) * w2               (blocks with a feed-forward)

State of a sequence: its K / V pages (one cache per block: blocks may differ in head count and
sizes) and, per block, the x row of its last token (token shift), kept in a state slot that the
scheduler assigns. The serving engine drives this class exactly as it drives
:class:`~nv_genai_amd.models.llama.LlamaModel` (``forward`` on a step's token rows + ``logits``);
``AttnMeta`` carries the extra per-step row maps (``tok_seq``, ``shift_src``, ``state_rows``,
``state_slots``).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..parallel.dist import ParallelContext, get_context
from .config import BidasunConfig
from .llama import AttnMeta


class BidasunModel:
    stateful = True               # per-sequence state slots besides the KV pages
    uses_decode_workspace = False  # no split-K softmax partials: sigmoid weights just add up
    supports_step_graphs = False   # prefill / mixed steps run eagerly (decode steps are graphs)
    supports_prefix_cache = False  # a cached page carries no token-shift state

    def __init__(self, cfg: BidasunConfig, device="cuda", dtype=torch.bfloat16,
                 pctx: Optional[ParallelContext] = None, seed: int = 0,
                 weights: Optional[Dict[str, torch.Tensor]] = None, fp8: bool = False):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Bidasun runs in bfloat16 or float32")
        if fp8:
            raise NotImplementedError("FP8 projections cover the Llama-layout decoders")
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.p = pctx or get_context()
        if self.p.tp_size > 1 or self.p.pp_size > 1:
            raise NotImplementedError("Bidasun runs on one GPU per replica (no TP / PP split)")
        self.fp8 = False
        self.kv_dtype, self.kv_scales = "auto", (1.0, 1.0)
        self.sequence_parallel, self.sp_min_tokens, self.split_mixed, self.moe_ws = False, 0, False, None
        m0 = cfg.blocks[0].mixer
        self.hq, self.hkv, self.D = m0.heads, m0.kv_heads, m0.dim
        self.vocab_local = cfg.vocab_size
        self.k_cache: List[torch.Tensor] = []
        self.v_cache: List[torch.Tensor] = []
        self.shift_state: List[torch.Tensor] = []
        self.skinny = (self.device.type == "cuda" and dtype == torch.bfloat16 and ops.skinny.enabled())
        self.mfma_prefill = True   # MFMA attention kernels where they apply (bf16, head sizes 32 / 64 / 128)
        if weights is None:
            weights = random_weights(cfg, seed, dtype)
        self._load(weights)

    # ------------------------------------------------------------------ weights
    def _load(self, w: Dict[str, torch.Tensor]):
        cfg, dev, dt = self.cfg, self.device, self.dtype

        def mat(name):
            return w[name].to(dev, dt).contiguous()

        def vec(name, n):
            t = w[name].to(dev, torch.float32).contiguous()
            if t.numel() != n:
                raise ValueError(f"{name}: {t.numel()} elements, config says {n}")
            return t

        H = cfg.hidden
        self.embed, self.pos_table = mat("embed"), mat("pos")
        if self.embed.shape != (cfg.vocab_size, H) or self.pos_table.shape != (cfg.max_position, H):
            raise ValueError("embed / pos tables do not fit the config")
        self.layers: List[dict] = []
        for i, b in enumerate(cfg.blocks):
            p, m = f"l{i}.", b.mixer
            nq, nk, nv, ng = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim, m.heads * m.vdim
            L = {"spec": m, "nq": nq, "nk": nk, "nv": nv, "ng": ng,
                 "shift": vec(p + "shift", H),
                 # q | k | v | gate in one GEMM: all four read the shifted input
                 "wqkvg": torch.cat([mat(p + "mix.q"), mat(p + "mix.k"), mat(p + "mix.v"), mat(p + "mix.g")]).contiguous(),
                 "qn": vec(p + "mix.q.norm", nq), "kn": vec(p + "mix.k.norm", nk),
                 "r1": vec(p + "mix.r1", m.heads), "r2": vec(p + "mix.r2", m.heads), "pb": vec(p + "mix.pb", m.heads),
                 "wo": mat(p + "mix.o"), "norm1": vec(p + "norm1", H)}
            if L["wqkvg"].shape != (nq + nk + nv + ng, H) or L["wo"].shape != (H, ng):
                raise ValueError(f"layer {i}: projection shapes do not fit the config")
            if b.mlp is not None:
                L["wgu"] = torch.cat([mat(p + "mlp.gate"), mat(p + "mlp.up")]).contiguous()
                L["wd"] = mat(p + "mlp.down")
                L["norm2"] = vec(p + "norm2", H)
                if L["wgu"].shape != (2 * b.mlp.ff, H) or L["wd"].shape != (H, b.mlp.ff):
                    raise ValueError(f"layer {i}: feed-forward shapes do not fit the config")
            self.layers.append(L)
        self.final_norm = vec("final.norm", H)
        self.lm_head = mat("head")

    def state_dict(self) -> Dict[str, torch.Tensor]:
        out = {"embed": self.embed, "pos": self.pos_table, "final.norm": self.final_norm.to(self.dtype),
               "head": self.lm_head}
        for i, L in enumerate(self.layers):
            p = f"l{i}."
            nq, nk, nv = L["nq"], L["nk"], L["nv"]
            W = L["wqkvg"]
            out.update({p + "mix.q": W[:nq], p + "mix.k": W[nq:nq + nk], p + "mix.v": W[nq + nk:nq + nk + nv],
                        p + "mix.g": W[nq + nk + nv:], p + "mix.o": L["wo"]})
            for k, n in (("shift", "shift"), ("qn", "mix.q.norm"), ("kn", "mix.k.norm"), ("r1", "mix.r1"),
                         ("r2", "mix.r2"), ("pb", "mix.pb"), ("norm1", "norm1")):
                out[p + n] = L[k].to(self.dtype)
            if "wgu" in L:
                F = L["wgu"].shape[0] // 2
                out.update({p + "mlp.gate": L["wgu"][:F], p + "mlp.up": L["wgu"][F:], p + "mlp.down": L["wd"],
                            p + "norm2": L["norm2"].to(self.dtype)})
        return out

    # ------------------------------------------------------------------ cache and state
    def allocate_kv_cache(self, num_blocks: int, block_size: int = 64, kv_dtype: str = "auto",
                          kv_scales=(1.0, 1.0)):
        """One paged cache per block: K [blocks, Hkv, 64, dim] and V^T [blocks, Hkv, vdim, 64]
        in the model dtype, all addressed by the same page numbers."""
        if block_size != 64:
            raise ValueError("the gfx950 attention kernels use 64-token KV pages")
        if kv_dtype not in ("auto", "bf16"):
            raise ValueError("Bidasun keeps its KV pages in the model dtype")
        self.k_cache, self.v_cache = [], []
        for L in self.layers:
            m = L["spec"]
            self.k_cache.append(torch.zeros(num_blocks, m.kv_heads, block_size, m.dim, device=self.device,
                                            dtype=self.dtype))
            self.v_cache.append(torch.zeros(num_blocks, m.kv_heads, m.vdim, block_size, device=self.device,
                                            dtype=self.dtype))
        return self.k_cache, self.v_cache

    def allocate_state(self, slots: int) -> None:
        """Token-shift state: per block one fp32 x row per slot. A slot needs no clearing when it
        is given to a new sequence: position 0 reads zeros, not the slot."""
        self.shift_state = [torch.zeros(max(1, slots), self.cfg.hidden, device=self.device, dtype=torch.float32)
                            for _ in self.layers]

    def kv_block_bytes(self, block_size: int = 64, kv_dtype: str = "auto") -> int:
        elem = torch.finfo(self.dtype).bits // 8
        return sum(b.mixer.kv_heads * (b.mixer.dim + b.mixer.vdim) for b in self.cfg.blocks) * block_size * elem

    def copy_kv_blocks(self, src, dst) -> None:
        raise NotImplementedError("beam search forks need a copy of the token-shift state")

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

    def _mixer(self, li: int, h, pos, meta: AttnMeta):
        L = self.layers[li]
        m = L["spec"]
        nq, nk, nv = L["nq"], L["nk"], L["nv"]
        proj = self._lin(h, L["wqkvg"])
        ops.qk_norm_cache_(proj, L["qn"], L["kn"], self.cfg.eps, meta.slots, self.k_cache[li], self.v_cache[li],
                           m.heads, m.kv_heads, m.dim, m.vdim)
        q, gate = proj[:, :nq], proj[:, nq + nk + nv:]
        kc, vc = self.k_cache[li], self.v_cache[li]
        args = (m.heads, m.kv_heads, m.dim, m.vdim, m.scale, m.window, m.keep_first, L["r1"], L["r2"], L["pb"])
        nd = meta.n_decode if meta.kind == "mixed" else 0
        if meta.kind in ("prefill", "mixed") and self.mfma_prefill and ops.sigmoid_attention_mfma_ok(proj, m.dim, m.vdim):
            # prompt portions on MFMA tiles; the single-token rows of a mixed step (its first
            # n_decode rows) on the row kernel, into disjoint rows of one output
            a = torch.empty(proj.shape[0], L["ng"], dtype=proj.dtype, device=proj.device)
            if nd:
                ops.sigmoid_attention_rows(q[:nd], gate[:nd], kc, vc, meta.block_tables, meta.tok_seq[:nd], pos[:nd],
                                           *args, max_ctx=meta.max_ctx, out=a[:nd])
            ops.sigmoid_attention_prefill(q[nd:], gate[nd:], kc, vc, meta.block_tables[nd:],
                                          meta.cu_q_prefill if nd else meta.cu_q, meta.ctx_lens[nd:],
                                          meta.max_q_len, *args, out=a[nd:])
        elif meta.kind == "decode" and self.mfma_prefill:
            a = ops.sigmoid_attention_rows(q, gate, kc, vc, meta.block_tables, meta.tok_seq, pos, *args,
                                           max_ctx=meta.max_ctx)
        else:
            a = ops.sigmoid_attention(q, gate, kc, vc, meta.block_tables, meta.tok_seq, pos, *args)
        return self._lin(a, L["wo"])

    def forward(self, ids: torch.Tensor, pos: torch.Tensor, meta: AttnMeta,
                sample_idx: Optional[torch.Tensor] = None, embed_override=None,
                layer_tap: Optional[list] = None) -> torch.Tensor:
        """Final-normed rows selected by ``sample_idx`` (all rows if None) of a step's token rows.
        ``layer_tap``: a list that receives a copy of the residual stream after every block."""
        if embed_override is not None:
            raise NotImplementedError("Bidasun takes token ids only")
        if meta.tok_seq is None or meta.shift_src is None:
            raise ValueError("Bidasun steps need the engine's row maps (tok_seq, shift_src, state rows)")
        eps = self.cfg.eps
        x = ops.embed_pos(ids, pos, self.embed, self.pos_table)
        T, H = x.shape
        for li, L in enumerate(self.layers):
            if meta.kind == "decode":   # one token per sequence: the shift kernel also leaves x in the slot
                h = ops.token_shift(x, L["shift"], meta.shift_src, self.shift_state[li], self.dtype,
                                    save_slots=meta.state_slots)
            else:
                h = ops.token_shift(x, L["shift"], meta.shift_src, self.shift_state[li], self.dtype)
                ops.shift_save_(self.shift_state[li], x, meta.state_rows, meta.state_slots)
            o = self._mixer(li, h, pos, meta)
            if "wgu" in L:
                xb = torch.empty(T, H, dtype=self.dtype, device=x.device)
                ops.rmsnorm_residual_(x, o, L["norm1"], eps, cast_out=xb)
                d = self._lin(ops.glu_gelu_tanh(self._lin(xb, L["wgu"])), L["wd"])
                ops.rmsnorm_residual_(x, d, L["norm2"], eps)
            else:
                ops.rmsnorm_residual_(x, o, L["norm1"], eps)
            if layer_tap is not None:
                layer_tap.append(x.clone())
        return ops.rmsnorm_f32(x, self.final_norm, eps, rows=sample_idx, dtype=self.dtype)

    def logits(self, h: torch.Tensor) -> torch.Tensor:
        return ops.linear(h, self.lm_head).float()


def random_weights(cfg: BidasunConfig, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random weights under the checkpoint's tensor names (benchmarks, tests, smoke runs)."""
    g = torch.Generator().manual_seed(seed)
    H = cfg.hidden

    def rnd(*shape, std):
        return (torch.randn(*shape, generator=g) * std).to(dtype)

    w = {"embed": rnd(cfg.vocab_size, H, std=1.0), "pos": rnd(cfg.max_position, H, std=0.3),
         "final.norm": (1.0 + 0.1 * torch.randn(H, generator=g)).to(dtype), "head": rnd(cfg.vocab_size, H, std=H ** -0.5)}
    for i, b in enumerate(cfg.blocks):
        p, m = f"l{i}.", b.mixer
        nq, nk, nv, ng = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim, m.heads * m.vdim
        s = H ** -0.5
        w.update({p + "shift": torch.rand(H, generator=g).to(dtype),
                  p + "mix.q": rnd(nq, H, std=s), p + "mix.k": rnd(nk, H, std=s), p + "mix.v": rnd(nv, H, std=s),
                  p + "mix.g": rnd(ng, H, std=s), p + "mix.o": rnd(H, ng, std=ng ** -0.5),
                  p + "mix.q.norm": (1.0 + 0.1 * torch.randn(nq, generator=g)).to(dtype),
                  p + "mix.k.norm": (1.0 + 0.1 * torch.randn(nk, generator=g)).to(dtype),
                  p + "mix.r1": (0.5 + torch.rand(m.heads, generator=g)).to(dtype),
                  p + "mix.r2": (0.05 + 0.5 * torch.rand(m.heads, generator=g)).to(dtype),
                  p + "mix.pb": (-1.0 + 0.5 * torch.randn(m.heads, generator=g)).to(dtype),
                  p + "norm1": (0.5 + 0.1 * torch.randn(H, generator=g)).to(dtype)})
        if b.mlp is not None:
            F = b.mlp.ff
            w.update({p + "mlp.gate": rnd(F, H, std=s), p + "mlp.up": rnd(F, H, std=s),
                      p + "mlp.down": rnd(H, F, std=F ** -0.5),
                      p + "norm2": (0.5 + 0.1 * torch.randn(H, generator=g)).to(dtype)})
    return w
