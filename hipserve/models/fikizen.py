"""Fikizen: a pre-norm layer-list decoder (``config.FikizenConfig``) on the hipserve op set.

    x <- x + mixer(norm1(x));   x <- x + ff(norm2(x))   (the second only where the layer has a feed-forward)

with the mixer one of ``models/mixers.py``: windowed sink attention with a per-head output
gate, a gated delta rule, or sink attention and a generalized delta rule side by side. A
layer may use another layer's weights; every layer RUN still has a paged cache and / or
state tensors of its own. The logits pass ``cap * tanh(. / cap)``.

The residual stream lives in 32-bit floats for every dtype; each residual update and the
norm that follows it are one fused op (``scaled_add_group_rmsnorm`` with one group). Per
engine step the model sees the flat token rows of all scheduled sequences (prompt portions
and single decode tokens alike); attention reads and writes the paged cache through the
step's block tables, the recurrences their sequences' state slots.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from ..config import FikizenConfig
from ..parallel.comm import TPGroup
from .mixers import DenseFF, make_mixer


class _Layer:
    def __init__(self):
        self.norm1 = self.norm2 = None   # [hidden] fp32
        self.mixer = None
        self.mlp = None


class FikizenModel:
    supports_fp32 = True        # every op of this model has a true 32-bit build
    graph_decode = True         # decode-only steps replay a captured hipGraph

    def __init__(self, cfg: FikizenConfig, tp: TPGroup, device, dtype=torch.bfloat16, ops=None,
                 max_pos: int | None = None):
        if tp.world_size != 1:
            raise NotImplementedError("the layer-list decoders run on one device (TP = 1)")
        self.cfg, self.tp, self.ops = cfg, tp, ops
        if hasattr(ops, "norm_library"):
            ops.norm_library = "delta"   # the residual + norm kernel from the library the mixers load
        self.device, self.dtype = torch.device(device), dtype
        self.kv_dtype = dtype
        self.vpad = cfg.vocab_size
        self.visual = None
        self.decode_partition = 512
        self.block_size_hint = 16
        self.runs = cfg.runs()
        # weight holders only for the layers that own weights
        self.layers: list[_Layer | None] = []
        H = cfg.hidden_size
        for spec in cfg.layers:
            if spec.weights_of is not None:
                self.layers.append(None)
                continue
            lw = _Layer()
            lw.mixer = make_mixer(spec.mixer, H, cfg.norm_eps, self.device, dtype, ops)
            if spec.mlp is not None:
                lw.mlp = DenseFF(spec.mlp, H, self.device, dtype, ops)
            self.layers.append(lw)
        self.embed = self.final_norm = self.lm_head = None
        self.capture = None  # a list: the residual stream after every layer run is appended (debugging)

    # ---------------------------------------------------------------- weights
    @property
    def needs_state(self) -> bool:
        return any(self.layers[i].mixer.state_shapes for i, _, _ in self.runs)

    def load_tensors(self, get):
        """``get(name)`` -> CPU tensor of the checkpoint (names: ``embed``, ``head``, ``final.norm``,
        ``l<i>.norm1`` / ``.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*`` for the layers with weights of their own)."""
        dev, dt = self.device, self.dtype
        self.embed = get("embed").to(dev, dt).contiguous()
        self.lm_head = get("head").to(dev, dt).contiguous()
        self.final_norm = get("final.norm").to(dev, torch.float32)
        for i, lw in enumerate(self.layers):
            if lw is None:
                continue
            lw.norm1 = get(f"l{i}.norm1").to(dev, torch.float32)
            lw.mixer.load(get, f"l{i}.mix.")
            if lw.mlp is not None:
                lw.norm2 = get(f"l{i}.norm2").to(dev, torch.float32)
                lw.mlp.load(get, f"l{i}.mlp.")

    def random_tensors(self, seed: int = 0, std: float = 0.05) -> dict:
        """Random checkpoint tensors (bf16-representable values) under the checkpoint's names."""
        cfg = self.cfg
        g = torch.Generator().manual_seed(seed)
        H, V = cfg.hidden_size, cfg.vocab_size
        out = {"embed": torch.randn(V, H, generator=g), "head": torch.randn(V, H, generator=g) * std * 4,
               "final.norm": 1.0 + 0.1 * torch.randn(H, generator=g)}
        for i, lw in enumerate(self.layers):
            if lw is None:
                continue
            out[f"l{i}.norm1"] = 1.0 + 0.1 * torch.randn(H, generator=g)
            for k, v in lw.mixer.init_random(g, std).items():
                out[f"l{i}.mix.{k}"] = v
            if lw.mlp is not None:
                out[f"l{i}.norm2"] = 1.0 + 0.1 * torch.randn(H, generator=g)
                for k, v in lw.mlp.init_random(g, std).items():
                    out[f"l{i}.mlp.{k}"] = v
        return {k: v.bfloat16().float() for k, v in out.items()}

    def allocate_random(self, seed: int = 0, std: float = 0.05):
        t = self.random_tensors(seed, std)
        self.load_tensors(lambda k: t[k])

    def allocate_random_quant(self, scheme: str, seed: int = 0):
        raise NotImplementedError("quantised weights are not available for this architecture")

    # ---------------------------------------------------------------- cache / state
    def _mixer(self, r: int):
        return self.layers[self.runs[r][0]].mixer

    def kv_bytes_per_block(self, block_size: int) -> int:
        el = torch.finfo(self.kv_dtype).bits // 8
        return max(1, sum(self._mixer(r).cache_dim for r in range(len(self.runs))) * block_size * el)

    def allocate_kv_cache(self, num_blocks: int, block_size: int):
        """One paged cache per layer RUN with attention: [num_blocks, block_size, all key heads | all value
        heads]; all runs share the sequences' block tables."""
        kv = [None] * len(self.runs)
        for r in range(len(self.runs)):
            n = self._mixer(r).cache_dim
            if n:
                kv[r] = torch.zeros(num_blocks, block_size, n, device=self.device, dtype=self.kv_dtype)
        return kv

    def state_bytes_per_slot(self) -> int:
        n = 0
        for r in range(len(self.runs)):
            f = self._mixer(r).state_shapes
            for shape in (f(1) if f else []):
                n += 4 * int(torch.tensor(shape).prod())
        return n

    def allocate_state(self, num_slots: int):
        """32-bit state tensors per layer run with a recurrence, indexed by sequence slot."""
        st = [None] * len(self.runs)
        for r in range(len(self.runs)):
            f = self._mixer(r).state_shapes
            if f:
                st[r] = [torch.zeros(shape, device=self.device, dtype=torch.float32) for shape in f(num_slots)]
        return st

    def step_workspace_bytes(self, tokens: int, seqs: int) -> int:
        el = torch.finfo(self.dtype).bits // 8
        wide = 0
        for lw in self.layers:
            if lw is None:
                continue
            n = 3 * sum(w.shape[0] for w in _in_weights(lw.mixer))
            if lw.mlp is not None:
                n = max(n, 2 * lw.mlp.spec.ff)
            wide = max(wide, n)
        return tokens * (wide * (el + 4) + 12 * self.cfg.hidden_size) + seqs * self.cfg.vocab_size * 12

    # ---------------------------------------------------------------- forward
    def forward(self, ids: torch.Tensor, meta, kv_caches) -> torch.Tensor:
        ops, cfg = self.ops, self.cfg
        T, H = ids.shape[0], cfg.hidden_size
        state = meta.state
        if meta.id_src is not None:  # decode lookahead: row i's id is the previous step's sample tok[src[i]]
            src, tok = meta.id_src
            ids = torch.where(src >= 0, tok.index_select(0, src.clamp(min=0)), ids)
        residual = F.embedding(ids, self.embed).to(torch.float32, copy=True)
        h = torch.empty(T, H, device=residual.device, dtype=self.dtype)
        first = self.layers[self.runs[0][0]].norm1 if self.runs else self.final_norm
        ops.scaled_add_group_rmsnorm(h, residual, first, 1, cfg.norm_eps)
        for r, (i, _, _) in enumerate(self.runs):
            lw = self.layers[i]
            mix = lw.mixer.forward(h, meta, kv_caches[r], state[r] if state is not None else None)
            nxt = self.final_norm if r + 1 == len(self.runs) else self.layers[self.runs[r + 1][0]].norm1
            hn = torch.empty_like(h)
            if lw.mlp is not None:
                ops.scaled_add_group_rmsnorm(hn, residual, lw.norm2, 1, cfg.norm_eps, mix)
                ff = lw.mlp.forward(hn)
                hn = torch.empty_like(h)
                ops.scaled_add_group_rmsnorm(hn, residual, nxt, 1, cfg.norm_eps, ff)
            else:
                ops.scaled_add_group_rmsnorm(hn, residual, nxt, 1, cfg.norm_eps, mix)
            if self.capture is not None:
                self.capture.append(residual.clone())
            h = hn
        return h

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """32-bit logits = cap * tanh(head . hidden / cap)."""
        if hidden.dtype == torch.float32:
            lg = F.linear(hidden, self.lm_head)
        elif hidden.is_cuda:
            lg = torch.mm(hidden, self.lm_head.t(), out_dtype=torch.float32)
        else:
            lg = F.linear(hidden.float(), self.lm_head.float())
        cap = self.cfg.logit_softcap
        return torch.tanh(lg / cap) * cap if cap > 0 else lg


def _in_weights(mixer):
    if hasattr(mixer, "left"):
        return _in_weights(mixer.left) + _in_weights(mixer.right)
    return [mixer.w_in]
