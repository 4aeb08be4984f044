"""Sequence mixers and feed-forwards of the layer-list decoders, as weight holders with a
``forward`` over the flat token rows of one engine step. Each is parameterised by its
spec (``config.LatentAttentionSpec`` / ``MinGRUSpec`` / ``TableMoESpec``) and runs on the
engine's op set (``ops.KernelOps`` on a GPU, ``ops.ReferenceOps`` on the CPU), so another
design can list them in its own layer order.

Dense projections are vendor GEMMs (``F.linear`` / ``torch.bmm``); everything between
them is one op of the op set:

* latent attention: merged [q-latent | kv-latent | rotary key | gate] projection ->
  ``latent_prepare`` (both latent RMSNorms, rotary key part, paged cache write) -> query
  up-projection -> per-head absorption of the key up-projection into the query (so the
  attention runs directly on the cached latents, one shared "key head" for all heads) ->
  ``latent_attention`` (rotary query part, sliding window, softmax, output gate) ->
  per-head value up-projection -> output projection.
* minGRU: merged [z | x | g] projection -> ``mingru_scan`` (gates, candidate, the
  recurrence over this step's tokens from the sequence's state slot, output gate) ->
  output projection.
* table MoE: expert ids looked up by token id -> ``moe_align`` tiles -> two
  ``expert_gemm`` launches (squared-ReLU in the first one's epilogue); the weighted
  combine is folded into the residual update (``scaled_add_group_rmsnorm``).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from ..config import LatentAttentionSpec, MinGRUSpec, TableMoESpec

MOE_TILE = 32        # slots per expert tile of the expert GEMMs ...
MOE_TILE_LARGE = 64  # ... when every expert has several tiles' worth of rows on average
# bf16 batches with at least this many (token, expert) pairs per expert run the packed-layout grouped
# GEMM of the dense families' MoE prefill (prefill_gemm_packed.hip: 128-row tiles, X through LDS, the
# weights pre-shuffled into MFMA operand order) with the squared ReLU in its epilogue
MOE_PACKED_MIN_PAIRS_PER_EXPERT = 256


def _mm32(x: torch.Tensor, w_t: torch.Tensor) -> torch.Tensor:
    """Batched product with a 32-bit result (the attention's query side stays 32-bit)."""
    if x.dtype == torch.float32:
        return torch.bmm(x, w_t)
    if x.is_cuda:
        return torch.bmm(x, w_t, out_dtype=torch.float32)
    return torch.bmm(x.float(), w_t.float())


class LatentAttention:
    def __init__(self, spec: LatentAttentionSpec, hidden: int, eps: float, device, dtype, ops):
        self.spec, self.hidden, self.eps, self.device, self.dtype, self.ops = spec, hidden, eps, device, dtype, ops
        s = spec
        self.w_in = None       # [q_rank + kv_rank + rot_dim + heads, hidden]
        self.q_norm = None     # [q_rank] fp32
        self.kv_norm = None    # [kv_rank] fp32
        self.w_uq = None       # [heads * (dim + rot_dim), q_rank]
        self.w_uk = None       # [heads, dim, kv_rank]
        self.w_uk_wide = None  # [heads, dim, kv_rank + rot_dim], zero rotary columns (made at first use)
        self.w_uv_t = None     # [heads, kv_rank, vdim]
        self.w_o = None        # [hidden, heads * vdim]
        rd = s.rot_dims or s.rot_dim
        i = torch.arange(rd // 2, dtype=torch.float32)
        # f_i = base^(-2i / dims), 32-bit
        self.inv_freq = torch.pow(torch.tensor(s.rot_base, dtype=torch.float32), -2.0 * i / rd).to(device)

    def load(self, get, prefix: str):
        s, dt, dev = self.spec, self.dtype, self.device
        self.w_in = torch.cat([get(prefix + "dq"), get(prefix + "dkv"), get(prefix + "g")], 0).to(dev, dt).contiguous()
        self.q_norm = get(prefix + "dq.norm").to(dev, torch.float32)
        self.kv_norm = get(prefix + "dkv.norm").to(dev, torch.float32)
        self.w_uq = get(prefix + "uq").to(dev, dt).contiguous()
        self.w_uk = get(prefix + "uk").to(dev, dt).view(s.heads, s.dim, s.kv_rank).contiguous()
        self.w_uv_t = get(prefix + "uv").to(dev, dt).view(s.heads, s.vdim, s.kv_rank).transpose(1, 2).contiguous()
        self.w_o = get(prefix + "o").to(dev, dt).contiguous()

    def init_random(self, gen, std: float):
        s, H = self.spec, self.hidden

        def w(*shape, scale=1.0):
            return torch.randn(*shape, generator=gen) * std * scale

        t = {"dq": w(s.q_rank, H), "dkv": w(s.key_dim, H), "g": w(s.heads, H),
             "dq.norm": 1.0 + 0.1 * torch.randn(s.q_rank, generator=gen),
             "dkv.norm": 1.0 + 0.1 * torch.randn(s.kv_rank, generator=gen),
             "uq": w(s.heads * (s.dim + s.rot_dim), s.q_rank, scale=4.0), "uk": w(s.heads * s.dim, s.kv_rank, scale=4.0),
             "uv": w(s.heads * s.vdim, s.kv_rank, scale=4.0), "o": w(H, s.heads * s.vdim)}
        self.load(lambda k: t[k], "")
        return t

    def cache_shape(self, num_blocks: int, block_size: int):
        return (num_blocks, block_size, self.spec.key_dim)

    def forward(self, h: torch.Tensor, meta, cache: torch.Tensor) -> torch.Tensor:
        s, ops = self.spec, self.ops
        T = h.shape[0]
        proj = F.linear(h, self.w_in)
        cq = torch.empty(T, s.q_rank, device=h.device, dtype=h.dtype)
        ops.latent_prepare(cq, cache, proj, meta.positions, meta.slot_mapping, self.q_norm, self.kv_norm,
                           self.inv_freq, s.q_rank, s.kv_rank, s.rot_dim, self.eps)
        q = F.linear(cq, self.w_uq)                                    # [T, heads * (dim + rot_dim)]
        qh = q.view(T, s.heads, s.dim + s.rot_dim)
        if ops.latent_query_in_place(h.dtype, s.kv_rank, s.rot_dim):
            # the absorption GEMM writes the attention kernel's query rows directly: bf16, the cached width,
            # zero weight columns where the attention op puts the rotated part
            if self.w_uk_wide is None:
                self.w_uk_wide = F.pad(self.w_uk, (0, s.rot_dim)).contiguous()
            q_abs = torch.bmm(qh[:, :, : s.dim].transpose(0, 1), self.w_uk_wide)   # [heads, T, kv_rank + rot_dim]
        else:
            q_abs = _mm32(qh[:, :, : s.dim].transpose(0, 1), self.w_uk)            # [heads, T, kv_rank] fp32
        o_lat = torch.empty(s.heads, T, s.kv_rank, device=h.device, dtype=h.dtype)
        ops.latent_attention(o_lat, q_abs, q, proj, cache, meta, self.inv_freq, s.heads, s.dim, s.rot_dim,
                             s.kv_rank, s.q_rank + s.key_dim, s.scale, s.window)
        o = torch.bmm(o_lat, self.w_uv_t)                              # [heads, T, vdim]
        return F.linear(o.transpose(0, 1).reshape(T, s.heads * s.vdim), self.w_o)


class MinGRU:
    def __init__(self, spec: MinGRUSpec, hidden: int, eps: float, device, dtype, ops):
        self.spec, self.hidden, self.device, self.dtype, self.ops = spec, hidden, device, dtype, ops
        self.w_in = None   # [3 * width, hidden]: z | x | g
        self.b_z = None    # [width] fp32
        self.b_x = None
        self.w_o = None    # [hidden, width]

    def load(self, get, prefix: str):
        dt, dev = self.dtype, self.device
        self.w_in = torch.cat([get(prefix + "z"), get(prefix + "x"), get(prefix + "g")], 0).to(dev, dt).contiguous()
        self.b_z = get(prefix + "z.b").to(dev, torch.float32)
        self.b_x = get(prefix + "x.b").to(dev, torch.float32)
        self.w_o = get(prefix + "o").to(dev, dt).contiguous()

    def init_random(self, gen, std: float):
        n, H = self.spec.width, self.hidden
        t = {k: torch.randn(n, H, generator=gen) * std * 4.0 for k in ("z", "x", "g")}
        t["z.b"] = torch.randn(n, generator=gen)
        t["x.b"] = torch.randn(n, generator=gen) * 0.5
        t["o"] = torch.randn(H, n, generator=gen) * std
        self.load(lambda k: t[k], "")
        return t

    def state_shape(self, num_slots: int):
        return (num_slots, self.spec.width)

    def forward(self, h: torch.Tensor, meta, state: torch.Tensor) -> torch.Tensor:
        proj = F.linear(h, self.w_in)
        y = torch.empty(h.shape[0], self.spec.width, device=h.device, dtype=h.dtype)
        self.ops.mingru_scan(y, state, proj, self.b_z, self.b_x, meta)
        return F.linear(y, self.w_o)


class TableMoE:
    """``forward`` returns (y [slots, hidden], pair_slot [T * top]): row ``pair_slot[t * top + j]``
    of ``y`` is token t's j-th expert output; the caller sums them with weight 1 / top."""

    def __init__(self, spec: TableMoESpec, hidden: int, vocab: int, device, dtype, ops):
        self.spec, self.hidden, self.vocab, self.device, self.dtype, self.ops = spec, hidden, vocab, device, dtype, ops
        self.table = None   # int32 [vocab, top]
        self.w_up = None    # [E, ff, hidden]
        self.w_down = None  # [E, hidden, ff]
        self.packed = None  # (up, down) in the packed grouped-GEMM layout, made at the first large batch

    def load(self, get, prefix: str):
        dt, dev, E = self.dtype, self.device, self.spec.experts
        self.table = get(prefix + "table").to(dev, torch.int32).contiguous()
        self.w_up = torch.stack([get(f"{prefix}e{e}.up") for e in range(E)]).to(dev, dt).contiguous()
        self.w_down = torch.stack([get(f"{prefix}e{e}.down") for e in range(E)]).to(dev, dt).contiguous()

    def init_random(self, gen, std: float):
        s, H = self.spec, self.hidden
        t = {"table": torch.stack([torch.randperm(s.experts, generator=gen)[: s.top] for _ in range(self.vocab)]).int()}
        for e in range(s.experts):
            t[f"e{e}.up"] = torch.randn(s.ff, H, generator=gen) * std * 4.0
            t[f"e{e}.down"] = torch.randn(H, s.ff, generator=gen) * std * 4.0
        self.load(lambda k: t[k], "")
        return t

    def forward(self, h: torch.Tensor, ids: torch.Tensor):
        s, ops = self.spec, self.ops
        T, dev = h.shape[0], h.device
        experts = self.table.index_select(0, ids).reshape(-1)          # [T * top]
        P = T * s.top
        if self._packed_ok(h, P):
            return self._forward_packed(h, experts, P)
        tile = MOE_TILE_LARGE if P >= 4 * MOE_TILE_LARGE * s.experts else MOE_TILE
        cap = -(-(P + s.experts * (tile - 1)) // tile) * tile
        slots = torch.empty(cap, dtype=torch.int32, device=dev)
        tile_expert = torch.empty(cap // tile, dtype=torch.int32, device=dev)
        pair_slot = torch.empty(P, dtype=torch.int32, device=dev)
        ops.moe_align(experts, s.experts, tile, slots, tile_expert, pair_slot)
        act = torch.empty(cap, s.ff, device=dev, dtype=h.dtype)
        ops.expert_gemm(act, h, self.w_up, slots, tile_expert, tile, s.top, True)
        y = torch.empty(cap, self.hidden, device=dev, dtype=h.dtype)
        ops.expert_gemm(y, act, self.w_down, slots, tile_expert, tile, 0, False)
        return y, pair_slot

    def _packed_ok(self, h: torch.Tensor, P: int) -> bool:
        s = self.spec
        return (getattr(self.ops, "name", "") == "hip" and h.dtype == torch.bfloat16 and s.experts <= 128
                and self.hidden % 256 == 0 and s.ff % 256 == 0
                and P >= MOE_PACKED_MIN_PAIRS_PER_EXPERT * s.experts and not torch.cuda.is_current_stream_capturing())

    def _forward_packed(self, h: torch.Tensor, experts: torch.Tensor, P: int):
        """Large bf16 batches: the experts as two launches of the packed-layout grouped GEMM (token rows
        gathered through the slot table inside the first one, squared ReLU in its epilogue)."""
        from ..ops import gemm

        s, dev = self.spec, h.device
        op = self.ops._op  # the core kernel library
        E, H, ff = s.experts, self.hidden, s.ff
        if self.packed is None:
            pu = torch.empty(E, -(-ff // 128) * 128 * H, dtype=h.dtype, device=dev)
            pd = torch.empty(E, -(-H // 128) * 128 * ff, dtype=h.dtype, device=dev)
            op.pack_decode_weight(pu, self.w_up, False)
            op.pack_decode_weight(pd, self.w_down, False)
            self.packed = (pu, pd)
        tile = 128 * gemm.PW_WM
        cap = -(-(P + E * (tile - 1)) // tile) * tile
        slots = torch.empty(cap, dtype=torch.int32, device=dev)
        tile_expert = torch.empty(cap // tile, dtype=torch.int32, device=dev)
        ntiles = torch.empty(1, dtype=torch.int32, device=dev)
        pair_slot = torch.empty(P, dtype=torch.int32, device=dev)
        op.moe_align(experts, E, tile, slots, tile_expert, ntiles, pair_slot, None)
        pu, pd = self.packed
        act = torch.empty(cap, ff, dtype=h.dtype, device=dev)
        op.prefill_gemm_packed_grouped(act, h, pu, ff, 4, tile_expert, ntiles, gemm.PW_WM, gemm.PW_RW, slots, s.top)
        y = torch.empty(cap, H, dtype=h.dtype, device=dev)
        op.prefill_gemm_packed_grouped(y, act, pd, H, 0, tile_expert, ntiles, gemm.PW_WM, gemm.PW_RW)
        return y, pair_slot
