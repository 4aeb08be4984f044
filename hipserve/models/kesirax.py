"""Kesirax: a layer-list decoder (``config.HybridConfig``) on the hipserve op set.

Every layer is a parallel block: one grouped RMSNorm feeds the sequence mixer (latent
attention or minGRU, ``models/mixers.py``) and the feed-forward (table-routed MoE), and
both results, each scaled per channel, are summed into the residual stream,

    x <- x + ls1 * mixer(norm(x)) + ls2 * ff(norm(x)).

A span of the layer list can run several passes with the same weights; every pass keeps
its own cache / state, and before each pass but the first the embedding output is added to
the stream again. The residual stream lives in 32-bit floats for every dtype; the update,
the MoE combine, the re-added embedding and the NEXT layer's norm are one fused op
(``scaled_add_group_rmsnorm``), as the add + RMSNorm of the other families.

Per engine step the model sees the flat token rows of all scheduled sequences (prompt
portions and single decode tokens alike); attention layers read and write the paged latent
cache through the step's block tables, recurrent layers their sequences' state slots.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from ..config import HybridConfig, LatentAttentionSpec, MinGRUSpec
from ..parallel.comm import TPGroup
from .mixers import LatentAttention, MinGRU, TableMoE


class _Layer:
    def __init__(self):
        self.norm = None    # [hidden] fp32
        self.mixer = None
        self.mlp = None
        self.ls1 = None     # [hidden] fp32
        self.ls2 = None


class KesiraxModel:
    supports_fp32 = True        # every op of this model has a true 32-bit build
    graph_decode = True         # decode-only steps replay a captured hipGraph

    def __init__(self, cfg: HybridConfig, tp: TPGroup, device, dtype=torch.bfloat16, ops=None,
                 max_pos: int | None = None):
        if tp.world_size != 1:
            raise NotImplementedError("the layer-list decoders run on one device (TP = 1)")
        self.cfg, self.tp, self.ops = cfg, tp, ops
        self.device, self.dtype = torch.device(device), dtype
        self.kv_dtype = dtype
        self.vpad = cfg.vocab_size
        self.visual = None
        self.decode_partition = 512
        self.block_size_hint = 16
        self.runs = cfg.runs()
        self.layers: list[_Layer] = []
        H = cfg.hidden_size
        for spec in cfg.layers:
            lw = _Layer()
            m = spec.mixer
            if isinstance(m, LatentAttentionSpec):
                lw.mixer = LatentAttention(m, H, cfg.norm_eps, self.device, dtype, ops)
            elif isinstance(m, MinGRUSpec):
                lw.mixer = MinGRU(m, H, cfg.norm_eps, self.device, dtype, ops)
            else:
                raise NotImplementedError(type(m).__name__)
            if spec.mlp is not None:
                lw.mlp = TableMoE(spec.mlp, H, cfg.vocab_size, self.device, dtype, ops)
            self.layers.append(lw)
        self.embed = self.final_norm = self.lm_head = None
        self.capture = None  # a list: the residual stream after every layer run is appended (debugging)

    # ---------------------------------------------------------------- weights
    @property
    def needs_state(self) -> bool:
        return any(isinstance(l.mixer, MinGRU) for l in self.layers)

    def load_tensors(self, get):
        """``get(name)`` -> CPU tensor of the checkpoint (names: ``embed``, ``head``,
        ``final.norm``, ``l<i>.norm1``, ``l<i>.ls1`` / ``.ls2``, ``l<i>.mix.*``, ``l<i>.mlp.*``)."""
        dev, dt = self.device, self.dtype
        self.embed = get("embed").to(dev, dt).contiguous()
        self.lm_head = get("head").to(dev, dt).contiguous()
        self.final_norm = get("final.norm").to(dev, torch.float32)
        for i, lw in enumerate(self.layers):
            lw.norm = get(f"l{i}.norm1").to(dev, torch.float32)
            lw.ls1 = get(f"l{i}.ls1").to(dev, torch.float32)
            lw.mixer.load(get, f"l{i}.mix.")
            if lw.mlp is not None:
                lw.ls2 = get(f"l{i}.ls2").to(dev, torch.float32)
                lw.mlp.load(get, f"l{i}.mlp.")

    def random_tensors(self, seed: int = 0, std: float = 0.05) -> dict:
        """Random checkpoint tensors (bf16-representable values) under the checkpoint's names."""
        cfg = self.cfg
        g = torch.Generator().manual_seed(seed)
        H, V = cfg.hidden_size, cfg.vocab_size
        out = {"embed": torch.randn(V, H, generator=g), "head": torch.randn(V, H, generator=g) * std,
               "final.norm": 1.0 + 0.1 * torch.randn(H, generator=g)}
        for i, lw in enumerate(self.layers):
            out[f"l{i}.norm1"] = 1.0 + 0.1 * torch.randn(H, generator=g)
            out[f"l{i}.ls1"] = 0.5 + 0.1 * torch.randn(H, generator=g)
            for k, v in lw.mixer.init_random(g, std).items():
                out[f"l{i}.mix.{k}"] = v
            if lw.mlp is not None:
                out[f"l{i}.ls2"] = 0.5 + 0.1 * torch.randn(H, generator=g)
                for k, v in lw.mlp.init_random(g, std).items():
                    out[f"l{i}.mlp.{k}"] = v
        return {k: (v if v.dtype == torch.int32 else v.bfloat16().float()) for k, v in out.items()}

    def allocate_random(self, seed: int = 0, std: float = 0.05):
        t = self.random_tensors(seed, std)
        self.load_tensors(lambda k: t[k])

    def allocate_random_quant(self, scheme: str, seed: int = 0):
        raise NotImplementedError("quantised weights are not available for this architecture")

    # ---------------------------------------------------------------- cache / state
    def _attn_runs(self):
        return [r for r, (i, _, _) in enumerate(self.runs) if isinstance(self.layers[i].mixer, LatentAttention)]

    def _state_runs(self):
        return [r for r, (i, _, _) in enumerate(self.runs) if isinstance(self.layers[i].mixer, MinGRU)]

    def kv_bytes_per_block(self, block_size: int) -> int:
        el = torch.finfo(self.kv_dtype).bits // 8
        return max(1, sum(self.layers[self.runs[r][0]].mixer.spec.key_dim for r in self._attn_runs()) * block_size * el)

    def allocate_kv_cache(self, num_blocks: int, block_size: int):
        """One paged latent cache per attention layer RUN (a looped layer has one per pass):
        [num_blocks, block_size, kv_rank + rot_dim]; all runs share the sequences' block tables."""
        kv = [None] * len(self.runs)
        for r in self._attn_runs():
            m = self.layers[self.runs[r][0]].mixer
            kv[r] = torch.zeros(m.cache_shape(num_blocks, block_size), device=self.device, dtype=self.kv_dtype)
        return kv

    def state_bytes_per_slot(self) -> int:
        return 4 * sum(self.layers[self.runs[r][0]].mixer.spec.width for r in self._state_runs())

    def allocate_state(self, num_slots: int):
        """Recurrent state per layer run and sequence slot, 32-bit: [num_slots, width]."""
        st = [None] * len(self.runs)
        for r in self._state_runs():
            m = self.layers[self.runs[r][0]].mixer
            st[r] = torch.zeros(m.state_shape(num_slots), device=self.device, dtype=torch.float32)
        return st

    def step_workspace_bytes(self, tokens: int, seqs: int) -> int:
        el = torch.finfo(self.dtype).bits // 8
        wide = 0
        for lw in self.layers:
            m = lw.mixer
            if isinstance(m, LatentAttention):
                s = m.spec
                n = 2 * (s.q_rank + s.key_dim + s.heads) + 2 * s.heads * (s.dim + s.rot_dim + s.vdim) + 6 * s.heads * s.kv_rank
            else:
                n = 5 * m.spec.width
            if lw.mlp is not None:
                n += 2 * lw.mlp.spec.top * (lw.mlp.spec.ff + self.cfg.hidden_size)
            wide = max(wide, n)
        return tokens * (wide * el + 12 * self.cfg.hidden_size) + seqs * self.cfg.vocab_size * 12

    # ---------------------------------------------------------------- forward
    def forward(self, ids: torch.Tensor, meta, kv_caches) -> torch.Tensor:
        ops, cfg = self.ops, self.cfg
        T, H = ids.shape[0], cfg.hidden_size
        state = meta.state
        if meta.id_src is not None:  # decode lookahead: row i's id is the previous step's sample tok[src[i]]
            src, tok = meta.id_src
            ids = torch.where(src >= 0, tok.index_select(0, src.clamp(min=0)), ids)
        x0 = F.embedding(ids, self.embed)                 # the embedding output (model dtype)
        residual = x0.to(torch.float32, copy=True)    # never an alias of x0 (float32 models)
        h = torch.empty(T, H, device=x0.device, dtype=self.dtype)
        first = self.layers[self.runs[0][0]] if self.runs else None
        ops.scaled_add_group_rmsnorm(h, residual, first.norm if first else self.final_norm, cfg.norm_groups, cfg.norm_eps)
        for r, (i, _, _) in enumerate(self.runs):
            lw = self.layers[i]
            if isinstance(lw.mixer, LatentAttention):
                mix = lw.mixer.forward(h, meta, kv_caches[r])
            else:
                mix = lw.mixer.forward(h, meta, state[r])
            y = pair_slot = None
            top = 0
            if lw.mlp is not None:
                y, pair_slot = lw.mlp.forward(h, ids)
                top = lw.mlp.spec.top
            last = r + 1 == len(self.runs)
            nxt = self.final_norm if last else self.layers[self.runs[r + 1][0]].norm
            extra = x0 if (not last and self.runs[r + 1][2]) else None
            hn = torch.empty_like(h)
            if self.capture is not None and extra is not None:
                ops.scaled_add_group_rmsnorm(hn, residual, nxt, cfg.norm_groups, cfg.norm_eps, mix, lw.ls1,
                                             y, pair_slot, top, lw.ls2)
                self.capture.append(residual.clone())
                ops.scaled_add_group_rmsnorm(hn, residual, nxt, cfg.norm_groups, cfg.norm_eps, extra=extra)
            else:
                ops.scaled_add_group_rmsnorm(hn, residual, nxt, cfg.norm_groups, cfg.norm_eps, mix, lw.ls1,
                                             y, pair_slot, top, lw.ls2, extra=extra)
                if self.capture is not None:
                    self.capture.append(residual.clone())
            h = hn
        return h

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """32-bit logits = head . hidden * logit_scale."""
        if hidden.dtype == torch.float32:
            lg = F.linear(hidden, self.lm_head)
        elif hidden.is_cuda:
            lg = torch.mm(hidden, self.lm_head.t(), out_dtype=torch.float32)
        else:
            lg = F.linear(hidden.float(), self.lm_head.float())
        return lg * self.cfg.logit_scale
