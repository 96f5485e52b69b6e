"""Layer-list decoders: every layer names its token mixer (windowed attention with a softmax
sink, the Mamba-2 recurrence, or latent attention) and an optional feed-forward; a span of layers
may run several times with shared weights.  ``Dunesun`` and ``Kisutar`` are the designs served;
mixers are registered by name (``MIXERS``) and feed-forward families by the design's ``ffn`` trait
(``FFNS``), with their sizes and constants read from the layer's spec, so another layer-list
design can reuse them in another order.  What a design fixes (block form, norm form, positions,
token shift, depth average) is models/config.DESIGN_TRAITS.

Kisutar, per layer (sequential block): ``x += mixer(shift(norm1(x)))``, then ``x += ff(norm2(x))``.
``shift`` moves every row towards the previous token's (per-channel learned fractions; the last
row of a sequence is state, one [d] fp32 vector per layer run and sequence slot).  The input of
layer i + 1 is a learned combination of the embedding output and the results of layers 0 .. i
(ops.hybrid.depth_mix; the results live in one fp32 stack [layers + 2, T, d]).  Its mixer is
latent attention: queries through a normed low-rank bottleneck; keys and values expanded per head
from one normed latent per token plus one rotated key part shared by all heads - only those two
are cached, and the per-head expansions are moved to the query side (the unrotated query is
multiplied into the latent space, the attention runs over the latent pages as one shared
key/value head, and the result is expanded to the value size afterwards), so prompt chunks and
decoding use the same pages and kernels as windowed attention.  A layer may read another layer's
pages (``kv_from``) with its own expansions.

Dunesun, per layer (parallel block): ``h = norm(x); x += mixer(h) + ff(h)`` with one one-plus
RMSNorm feeding both branches.  The residual stream is fp32 whatever the activation dtype, and the
branch sums of layer i are folded into layer i+1's norm launch (ops.hybrid.add_norm), like the
fused add + RMSNorm of the Llama path.  Looped layers: pass t starts with ``x += loop.step[t]``
(and ``x += embedding output`` for t > 0), folded into the same launch.

State: an attention run owns paged K ``[blocks, 16, heads*dim]`` and V ``[blocks, heads, vdim, 16]``
(activation dtype); a
Mamba-2 run owns per-sequence slots - the fp32 state ``[slots, heads, N, P]`` and the last
taps-1 convolution inputs.  Every RUN (a looped layer counts once per pass) has its own.

Dense projections go to the BLAS library (``F.linear``); everything else is ops.hybrid.
"""
from __future__ import annotations

import hashlib
import math
from typing import Optional

import torch
import torch.nn.functional as F

from .. import ops as _ops
from ..ops import hybrid as hops
from ..parallel.state import ParallelState, get_state
from .config import DenseSpec, HybridConfig, LayerSpec, MoESpec
from .llama import AttnMeta

BLOCK = 16  # tokens per cache page (engine/runner.BLOCK_SIZE)


def _seed_for(name: str, seed: int) -> int:
    h = hashlib.blake2b(f"{seed}:{name}".encode(), digest_size=8).digest()
    return int.from_bytes(h, "little") & 0x7FFF_FFFF_FFFF_FFFF


class _Params:
    """Creates a model's tensors: seeded random values per checkpoint name, or the checkpoint's."""

    def __init__(self, device, dtype, seed: int, src=None, empty: bool = False):
        self.device, self.dtype, self.seed, self.src, self.empty = device, dtype, seed, src, empty
        self.used: set = set()

    def get(self, name: str, shape: tuple, std: float = 0.02, mean: float = 0.0, small: bool = False) -> torch.Tensor:
        """``small``: a vector or table the kernels read as fp32, kept fp32 on the device."""
        dt = torch.float32 if small else self.dtype
        if self.src is not None:
            t = self.src.get(name)
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: checkpoint shape {tuple(t.shape)}, config says {tuple(shape)}")
            self.used.add(name)
            return t.to(self.device, dt).contiguous()
        if self.empty:
            return torch.empty(shape, dtype=dt, device=self.device)
        g = torch.Generator().manual_seed(_seed_for(name, self.seed))
        t = torch.randn(shape, generator=g) * std + mean
        return t.to(torch.bfloat16).to(self.device, dt).contiguous()  # values a bf16 checkpoint could hold


class WindowAttention:
    """Grouped-query attention with a whole-projection RMSNorm of q and of k, no positional
    rotation, a sliding window of ``mask.size`` keys (0 / absent: unbounded) and a softmax sink."""

    kind = "attention"

    def __init__(self, spec: LayerSpec, d: int, eps: float, p: _Params, prefix: str):
        m = spec.m
        self.H, self.G, self.dk, self.dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        if self.H % self.G:
            raise ValueError(f"{prefix}: heads {self.H} not a multiple of kv_heads {self.G}")
        self.scale = float(m.get("scale", 1.0 / math.sqrt(self.dk)))
        self.window = int(m.get("mask.size", 0) or 0)
        self.sink = bool(m.get("sink", True))
        self.eps = eps
        self.fast = 1  # 0: the any-size attention kernels only (ops.hybrid mfma / vec switches; tests)
        nq, nk, nv = self.H * self.dk, self.G * self.dk, self.G * self.dv
        s = 1.0 / math.sqrt(d)
        self.wqkv = torch.cat([p.get(prefix + "q", (nq, d), s), p.get(prefix + "k", (nk, d), s),
                               p.get(prefix + "v", (nv, d), s)]).contiguous()
        self.qn = p.get(prefix + "q.norm", (nq,), 0.1, 1.0, small=True)
        self.kn = p.get(prefix + "k.norm", (nk,), 0.1, 1.0, small=True)
        self.wo = p.get(prefix + "o", (d, self.H * self.dv), 1.0 / math.sqrt(self.H * self.dv))

    def new_cache(self, num_blocks: int, num_slots: int, dtype, device) -> dict:
        return {"k": torch.zeros(num_blocks, BLOCK, self.G * self.dk, dtype=dtype, device=device),
                "v": torch.zeros(num_blocks, self.G, self.dv, BLOCK, dtype=dtype, device=device)}

    def cache_bytes(self, esize: int) -> tuple:
        """(bytes per page, bytes per state slot)."""
        return BLOCK * self.G * (self.dk + self.dv) * esize, 0

    def forward(self, h: torch.Tensor, meta: AttnMeta, cache: dict) -> torch.Tensor:
        H, G, dk, dv = self.H, self.G, self.dk, self.dv
        qkv = F.linear(h, self.wqkv)
        kc, vc = cache["k"], cache["v"]
        hops.qk_norm_cache(qkv, self.qn, self.kn, self.eps, H, G, dk, dv, kc, vc, meta.slot_mapping)
        args = (H, G, dk, dv, self.scale, self.window, self.sink)
        if not meta.is_prefill:
            o = hops.window_attention_decode(qkv, kc, vc, meta.block_tables, meta.seq_lens, *args, vec=bool(self.fast))
        else:
            nd = meta.num_decode
            o = hops.window_attention_prefill(qkv[nd:], kc, vc, meta.cu_seqlens, meta.ctx_start, meta.block_tables,
                                              *args, mfma=self.fast)
            if nd:  # a mixed step: the single decode tokens in front go through the decode kernel
                od = hops.window_attention_decode(qkv[:nd], kc, vc, meta.dec_block_tables, meta.dec_seq_lens, *args,
                                                  vec=bool(self.fast))
                o = torch.cat([od, o])
        return F.linear(o, self.wo)


class Mamba2Mixer:
    """Mamba-2 (state-space duality) mixer: in-projection [z | x | B | C | dt], short causal
    convolution + SiLU over x, B, C, the fp32 recurrence per head, gate then grouped RMSNorm, and
    the out-projection."""

    kind = "mamba2"

    def __init__(self, spec: LayerSpec, d: int, eps: float, p: _Params, prefix: str):
        m = spec.m
        self.nh, self.P, self.N = int(m["heads"]), int(m["vdim"]), int(m["state"])
        self.G, self.taps, self.ng = int(m.get("groups", 1)), int(m["conv"]), int(m.get("norm_groups", 1))
        self.inner = self.nh * self.P
        self.C = self.inner + 2 * self.G * self.N
        if self.nh % self.G or self.inner % self.ng or self.taps < 1:
            raise ValueError(f"{prefix}: heads/groups/norm_groups/conv do not fit")
        self.eps = eps
        self.w_in = p.get(prefix + "in", (self.inner + self.C + self.nh, d), 1.0 / math.sqrt(d))
        self.conv_w = p.get(prefix + "conv", (self.C, self.taps), 0.4, small=True)
        self.conv_b = p.get(prefix + "conv.b", (self.C,), 0.1, small=True)
        self.dt_bias = p.get(prefix + "dt_bias", (self.nh,), 0.5, -1.0, small=True)
        self.a_log = p.get(prefix + "A_log", (self.nh,), 0.5, -0.5, small=True)
        self.d_skip = p.get(prefix + "D", (self.nh,), 0.3, 1.0, small=True)
        self.norm_w = p.get(prefix + "norm", (self.inner,), 0.1, 1.0, small=True)
        self.wo = p.get(prefix + "o", (d, self.inner), 1.0 / math.sqrt(self.inner))

    def new_cache(self, num_blocks: int, num_slots: int, dtype, device) -> dict:
        return {"conv": torch.zeros(num_slots, max(1, self.taps - 1), self.C, dtype=dtype, device=device),
                "ssm": torch.zeros(num_slots, self.nh, self.N, self.P, dtype=torch.float32, device=device)}

    def cache_bytes(self, esize: int) -> tuple:
        return 0, (self.taps - 1) * self.C * esize + self.nh * self.N * self.P * 4

    def forward(self, h: torch.Tensor, meta: AttnMeta, cache: dict) -> torch.Tensor:
        proj = F.linear(h, self.w_in)
        seg = (meta.seg_cu, meta.seg_ctx, meta.seg_slot)
        xbc = hops.conv_silu(proj, self.inner, self.C, self.conv_w, self.conv_b, cache["conv"], *seg)
        y = hops.ssm_scan(xbc, proj, self.inner + self.C, self.dt_bias, self.a_log, self.d_skip, cache["ssm"], *seg,
                          self.nh, self.P, self.N, self.G)
        g = hops.gated_group_norm(y, proj, 0, self.norm_w, self.eps, self.ng, h.dtype)
        return F.linear(g, self.wo)


class LatentAttention:
    """Attention over a compressed key/value stream (one normed latent of ``kv_rank`` and one
    rotated key part of ``rot_dim`` per token, shared by all heads), rotary positions on the
    ``rot_dim`` part of queries and keys, a sliding window and a learned per-head sink.
    ``kv_from``: j - no key/value projection of its own; reads layer j's pages."""

    kind = "latent_attention"

    def __init__(self, spec: LayerSpec, d: int, eps: float, p: _Params, prefix: str):
        m = spec.m
        self.H, self.dn, self.dr, self.dv = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
        self.Q, self.R = int(m["q_rank"]), int(m["kv_rank"])
        self.scale = float(m.get("scale", 1.0 / math.sqrt(self.dn + self.dr)))
        self.window = int(m.get("mask.size", 0) or 0)
        self.base, self.rdims = float(m.get("rot.base", 10000.0)), int(m.get("rot.dims", self.dr))
        if self.rdims % 2 or self.rdims > self.dr:
            raise ValueError(f"{prefix}: rot.dims {self.rdims} must be even and at most rot_dim {self.dr}")
        self.kv_from = m.get("kv_from")
        self.kv_from = None if self.kv_from is None else int(self.kv_from)
        self.eps = eps
        self.fast = 1
        self.pitch = (self.R + self.dr + 31) // 32 * 32
        H, dn, dr, dv, Q, R = self.H, self.dn, self.dr, self.dv, self.Q, self.R
        wd = [p.get(prefix + "dq", (Q, d), 1.0 / math.sqrt(d))]
        self.kn = None
        if self.kv_from is None:
            wd.append(p.get(prefix + "dkv", (R + dr, d), 1.0 / math.sqrt(d)))
            self.kn = p.get(prefix + "dkv.norm", (R,), 0.1, 1.0, small=True)
        self.w_down = torch.cat(wd).contiguous()  # [q_rank (+ kv_rank + rot_dim), d]: one launch
        self.qn = p.get(prefix + "dq.norm", (Q,), 0.1, 1.0, small=True)
        self.w_uq = p.get(prefix + "uq", (H * (dn + dr), Q), 1.0 / math.sqrt(Q))
        self.w_uk = p.get(prefix + "uk", (H * dn, R), 1.0 / math.sqrt(R))  # viewed [H, dn, R]
        self.w_uv = p.get(prefix + "uv", (H * dv, R), 1.0 / math.sqrt(R))  # viewed [H, dv, R]
        self.sinks = p.get(prefix + "sink", (H,), 1.0, small=True)
        self.freq = hops.rotary_freq(self.base, self.rdims, p.device)
        self.wo = p.get(prefix + "o", (d, H * dv), 1.0 / math.sqrt(H * dv))

    def new_cache(self, num_blocks: int, num_slots: int, dtype, device) -> dict:
        if self.kv_from is not None:
            return {}
        # key rows [latent | rotated part], padded with zeros to the matrix-core kernel's multiple of 32
        return {"k": torch.zeros(num_blocks, BLOCK, self.pitch, dtype=dtype, device=device),
                "v": torch.zeros(num_blocks, 1, self.R, BLOCK, dtype=dtype, device=device)}

    def cache_bytes(self, esize: int) -> tuple:
        return (0 if self.kv_from is not None else BLOCK * (self.pitch + self.R) * esize), 0

    def forward(self, h: torch.Tensor, meta: AttnMeta, cache: dict) -> torch.Tensor:
        H, dn, dr, dv, Q, R = self.H, self.dn, self.dr, self.dv, self.Q, self.R
        T = h.shape[0]
        down = F.linear(h, self.w_down)
        kc, vc = cache["k"], cache["v"]
        own = self.kv_from is None
        hops.latent_prep(down, Q, R, dr, self.qn, self.kn, self.eps, meta.positions, self.freq,
                         kc if own else None, vc if own else None, meta.slot_mapping if own else None)
        q = F.linear(down[:, :Q], self.w_uq)
        # the per-head key expansion moved to the query: q_lat[h] = q_unrotated[h] @ W_uk[h]  ([H, T, R])
        q_lat = torch.bmm(q.view(T, H, dn + dr)[:, :, :dn].transpose(0, 1), self.w_uk.view(H, dn, R))
        qa = hops.latent_queries(q, q_lat, H, dn, dr, meta.positions, self.freq, self.pitch)
        args = (H, self.scale, self.window, self.sinks)
        if not meta.is_prefill:
            o = hops.latent_attention(qa, kc, vc, meta.block_tables, *args, seq_lens=meta.seq_lens, fast=self.fast)
        else:
            nd = meta.num_decode
            o = hops.latent_attention(qa[nd:], kc, vc, meta.block_tables, *args, cu=meta.cu_seqlens, ctx=meta.ctx_start,
                                      fast=self.fast)
            if nd:
                od = hops.latent_attention(qa[:nd], kc, vc, meta.dec_block_tables, *args, seq_lens=meta.dec_seq_lens,
                                           fast=self.fast)
                o = torch.cat([od, o])
        # ... and the value expansion to the result: v[h] = o_lat[h] @ W_uv[h]^T, written head by head
        # into the rows the out-projection reads
        v = torch.empty(T, H, dv, dtype=h.dtype, device=h.device)
        torch.bmm(o.view(T, H, R).transpose(0, 1), self.w_uv.view(H, dv, R).transpose(1, 2), out=v.transpose(0, 1))
        return F.linear(v.view(T, H * dv), self.wo)


MIXERS = {WindowAttention.kind: WindowAttention, Mamba2Mixer.kind: Mamba2Mixer, LatentAttention.kind: LatentAttention}


class RoutedFFN:
    """Top-k routed SwiGLU experts (biased fp32 router, softmax over the chosen logits) plus an
    optional shared expert scaled by sigmoid of a per-token gate.  The gate's weight row rides as
    one more row of the router matrix, so router logits and gate come out of one launch."""

    def __init__(self, spec: MoESpec, d: int, p: _Params, prefix: str):
        self.E, self.K, self.ff, self.fs = spec.experts, spec.top, spec.ff, spec.shared_ff
        if not 1 <= self.K <= self.E:
            raise ValueError(f"{prefix}: top {self.K} of {self.E} experts")
        s, s2 = 1.0 / math.sqrt(d), 1.0 / math.sqrt(self.ff)
        # gate / up rows interleaved per 128 ([64 gate | 64 up]): the layout of the prefill tile GEMM's
        # SwiGLU epilogue, which large bf16 steps on the GPU use (ops.hybrid.moe_experts); ONE copy
        self.il = (p.device.type == "cuda" and p.dtype == torch.bfloat16 and self.ff % 128 == 0 and d % 128 == 0)
        pair = _ops.interleave_gate_up if self.il else (lambda w: w)
        self.w13 = torch.stack([pair(torch.cat([p.get(f"{prefix}e{e}.gate", (self.ff, d), s),
                                                p.get(f"{prefix}e{e}.up", (self.ff, d), s)])) for e in range(self.E)])
        self.w2 = torch.stack([p.get(f"{prefix}e{e}.down", (d, self.ff), s2) for e in range(self.E)])
        wr = p.get(prefix + "router", (self.E, d), 2 * s, small=True)
        self.bias = p.get(prefix + "router.b", (self.E,), 0.2, small=True)
        self.ws13 = self.ws2 = None
        if self.fs:
            self.ws13 = torch.cat([p.get(prefix + "shared.gate", (self.fs, d), s),
                                   p.get(prefix + "shared.up", (self.fs, d), s)]).contiguous()
            self.ws2 = p.get(prefix + "shared.down", (d, self.fs), 1.0 / math.sqrt(self.fs))
            wr = torch.cat([wr, p.get(prefix + "shared.sg", (1, d), s, small=True)])
        self.wr = wr.contiguous()

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ids, wts, gate = hops.moe_router(h, self.wr, self.bias, self.E, self.K)
        shared = None
        if self.fs:
            shared = F.linear(hops.swiglu(F.linear(h, self.ws13)), self.ws2)
        return hops.moe_experts(h, ids, wts, self.w13, self.w2, shared, gate, il=self.il)


def _softplus(z: float) -> float:
    return z if z > 30.0 else math.log1p(math.exp(z))


class DenseFFN:
    """``down(xIELU(up h))``; the activation's two constants come from the two learned numbers of
    ``act`` (softplus of the first; one half plus softplus of the second), evaluated once at load."""

    def __init__(self, spec: DenseSpec, d: int, p: _Params, prefix: str):
        self.ff = spec.ff
        self.w_up = p.get(prefix + "up", (self.ff, d), 1.0 / math.sqrt(d))
        self.w_down = p.get(prefix + "down", (d, self.ff), 1.0 / math.sqrt(self.ff))
        self.act = p.get(prefix + "act", (2,), 0.5, small=True)
        a = self.act.float().cpu().tolist() if not p.empty else [0.0, 0.0]
        self.a_pos, self.a_neg = _softplus(a[0]), 0.5 + _softplus(a[1])

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(hops.activation(F.linear(h, self.w_up), "xielu", self.a_pos, self.a_neg), self.w_down)


class PlainRoutedFFN:
    """Top-k routed ungated experts ``down_e(gelu(up_e h))`` (erf GELU): fp32 router without bias,
    softmax over all experts, the chosen experts weighted by their probabilities as they are; plus
    an optional shared expert of the same form, added for every token."""

    def __init__(self, spec: MoESpec, d: int, p: _Params, prefix: str):
        self.E, self.K, self.ff, self.fs = spec.experts, spec.top, spec.ff, spec.shared_ff
        if not 1 <= self.K <= self.E:
            raise ValueError(f"{prefix}: top {self.K} of {self.E} experts")
        s, s2 = 1.0 / math.sqrt(d), 1.0 / math.sqrt(self.ff)
        self.il = False
        # large bf16 steps of such experts run on the Mixtral path's tile GEMM (ops.hybrid.moe_experts)
        self.tile = p.device.type == "cuda" and p.dtype == torch.bfloat16 and self.ff % 256 == 0 and d % 256 == 0
        self.w1 = torch.stack([p.get(f"{prefix}e{e}.up", (self.ff, d), s) for e in range(self.E)])
        self.w2 = torch.stack([p.get(f"{prefix}e{e}.down", (d, self.ff), s2) for e in range(self.E)])
        self.wr = p.get(prefix + "router", (self.E, d), 2 * s, small=True)
        self.ws1 = self.ws2 = None
        if self.fs:
            self.ws1 = p.get(prefix + "shared.up", (self.fs, d), s)
            self.ws2 = p.get(prefix + "shared.down", (d, self.fs), 1.0 / math.sqrt(self.fs))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ids, wts, _ = hops.moe_router(h, self.wr, None, self.E, self.K, over_all=True)
        shared = None
        if self.fs:
            shared = F.linear(hops.activation(F.linear(h, self.ws1), "gelu"), self.ws2)
        return hops.moe_experts(h, ids, wts, self.w1, self.w2, shared, None, act="gelu")


def _ffn_for(family: str, spec, d: int, p: _Params, prefix: str):
    """The feed-forward of a layer in a design's family (models/config.DESIGN_TRAITS ``ffn``)."""
    if spec is None:
        return None
    if family == "swiglu_topk" and isinstance(spec, MoESpec):
        return RoutedFFN(spec, d, p, prefix)
    if family == "plain_softmax":
        return DenseFFN(spec, d, p, prefix) if isinstance(spec, DenseSpec) else PlainRoutedFFN(spec, d, p, prefix)
    raise ValueError(f"{prefix}: no {type(spec).__name__} feed-forward in the {family!r} family")


class HybridLM:
    """The model class of layer-list configs (models/registry.py).  TP = 1."""

    def __init__(self, cfg: HybridConfig, device: torch.device | str = "cpu", dtype=torch.bfloat16, seed: int = 0,
                 pstate: Optional[ParallelState] = None, init: str = "random", weights=None):
        """``weights``: a models/checkpoint.SafetensorsDir to read the tensors from (names
        ``embed``, ``pos``, ``loop.step``, ``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.mlp.*``,
        ``final.norm``, ``head``); otherwise ``init`` "random" (seeded per name) or "empty"."""
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.seed = seed
        self.ps = pstate or get_state()
        if self.ps.tp_size != 1:
            raise ValueError(f"{cfg.name}: layer-list models run at tp=1")
        self.tp, self.rank = 1, 0
        d, V = cfg.d_model, cfg.vocab_size
        p = _Params(self.device, dtype, seed, src=weights, empty=init == "empty")
        tr = cfg.traits
        self.sequential = tr["block"] == "sequential"
        self.one_plus, self.shifted, self.depth_avg = tr["one_plus_norm"], tr["token_shift"], tr["depth_average"]
        if (self.shifted or self.depth_avg) and not self.sequential:
            raise ValueError(f"{cfg.name}: token shift and depth average are built for sequential blocks")
        if self.depth_avg and cfg.loop:
            raise ValueError(f"{cfg.name}: depth average over looped layers is not defined")
        nm = 1.0 if not self.one_plus else 0.0  # plain norm weights sit around one
        self.embed = p.get("embed", (V, d), 0.5)
        self.pos = p.get("pos", (cfg.max_position, d), 0.1) if tr["learned_pos"] else None
        self.loop_step = p.get("loop.step", (cfg.loop[2], d), 0.1, small=True) if cfg.loop else None
        self.norms, self.norms2, self.mixers, self.ffns, self.shifts, self.dwa = [], [], [], [], [], []
        for i, spec in enumerate(cfg.layers):
            if spec.kind not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer {spec.kind!r} (known: {sorted(MIXERS)})")
            self.norms.append(p.get(f"l{i}.norm1", (d,), 0.1, nm, small=True))
            self.mixers.append(MIXERS[spec.kind](spec, d, cfg.norm_eps, p, f"l{i}.mix."))
            self.ffns.append(_ffn_for(tr["ffn"], spec.mlp, d, p, f"l{i}.mlp."))
            self.norms2.append(p.get(f"l{i}.norm2", (d,), 0.1, nm, small=True)
                               if self.sequential and spec.mlp is not None else None)
            self.shifts.append(p.get(f"l{i}.shift", (d,), 0.25, 0.4, small=True) if self.shifted else None)
            # depth-average coefficients: random init leans on the newest result so the stream stays sane
            self.dwa.append(p.get(f"l{i}.dwa", (i + 2,), 0.3 / (i + 2), 1.0 / (i + 2), small=True)
                            if self.depth_avg else None)
        self.final_norm = p.get("final.norm", (d,), 0.1, nm, small=True)
        self.head = p.get("head", (V, d), 1.0 / math.sqrt(d))
        self.runs = cfg.runs()
        # the run whose pages a run reads: its own, or the latest earlier run of the layer it names
        self.kv_run = []
        for r, (li, _, _) in enumerate(self.runs):
            src = getattr(self.mixers[li], "kv_from", None)
            if src is None:
                self.kv_run.append(r)
                continue
            if not 0 <= src < len(cfg.layers) or getattr(self.mixers[src], "kv_from", 0) is not None:
                raise ValueError(f"layer {li}: kv_from {src} is not a layer with key/value pages of its own")
            a, b = self.mixers[li], self.mixers[src]
            if (a.R, a.dr, a.base, a.rdims) != (b.R, b.dr, b.base, b.rdims):
                raise ValueError(f"layer {li}: kv_rank / rot_dim / rotation differ from layer {src}'s")
            prev = [q for q in range(r) if self.runs[q][0] == src]
            if not prev:
                raise ValueError(f"layer {li}: kv_from {src} has not run before it")
            self.kv_run.append(prev[-1])
        self.unused = sorted(set(weights.keys()) - p.used) if weights is not None else []
        self.has_state = self.shifted or any(m.kind == "mamba2" for m in self.mixers)
        # large steps of such layers run on the Mixtral path's tile GEMM (extension _k8sllm_ops)
        self.uses_tile_gemm = any(f is not None and (getattr(f, "il", False) or getattr(f, "tile", False))
                                  for f in self.ffns)
        self.layer_probe = None  # a list: forward() appends the residual stream after every run

    # ------------------------------------------------------------------ engine interface
    def overlap_ok(self) -> bool:
        return False

    def cache_bytes(self) -> tuple:
        """(bytes per cache page, bytes per state slot) summed over the layer runs."""
        es = torch.empty(0, dtype=self.dtype).element_size()
        per = [self.mixers[i].cache_bytes(es) for i, _, _ in self.runs]
        shift = 4 * self.cfg.d_model * len(self.runs) if self.shifted else 0
        return sum(a for a, _ in per), sum(b for _, b in per) + shift

    def new_cache(self, num_blocks: int, num_slots: int) -> list:
        """One cache per layer RUN (a looped layer has one per pass): the mixer's pages or state
        slots and, with token shift, the run's last normed row per sequence slot (``shift``)."""
        out = []
        for i, _, _ in self.runs:
            c = self.mixers[i].new_cache(num_blocks, num_slots, self.dtype, self.device)
            if self.shifted:
                c["shift"] = torch.zeros(num_slots, self.cfg.d_model, dtype=torch.float32, device=self.device)
            out.append(c)
        return out

    def resident_weight_bytes(self) -> int:
        n = 0
        for t in self._tensors():
            n += t.numel() * t.element_size()
        return n

    def num_local_params(self) -> int:
        return sum(t.numel() for t in self._tensors())

    def _tensors(self) -> list:
        ts = [self.embed, self.final_norm, self.head] + self.norms
        ts += [t for t in [self.pos, self.loop_step] + self.norms2 + self.shifts + self.dwa if t is not None]
        for o in self.mixers + [f for f in self.ffns if f is not None]:
            ts += [v for v in vars(o).values() if isinstance(v, torch.Tensor)]
        return ts

    # ------------------------------------------------------------------ forward
    def forward(self, ids: torch.Tensor, meta: AttnMeta, caches: list) -> torch.Tensor:
        """Logits [rows, vocab] (fp32) for the rows ``meta.logits_idx`` selects (all when None)."""
        c = self.cfg
        if self.sequential:
            return self._forward_sequential(ids, meta, caches)
        x0 = hops.embed_pos(ids, meta.positions, self.embed, self.pos, meta.dec_src, meta.dec_prev)
        x = x0.clone() if c.loop and c.loop[2] > 1 else x0
        pending: tuple = ()
        for r, (li, t, first) in enumerate(self.runs):
            adds, vec = pending, None
            if first:
                vec = self.loop_step[t]
                if t > 0:
                    adds = adds + (x0,)
            h = hops.add_norm(x, adds, vec, self.norms[li], c.norm_eps, True, self.dtype)
            ym = self.mixers[li].forward(h, meta, caches[r])
            ff = self.ffns[li]
            pending = (ym, ff.forward(h)) if ff is not None else (ym,)
            if self.layer_probe is not None:
                self.layer_probe.append(x + sum(a.float() for a in pending))
        if meta.logits_idx is not None:
            idx = meta.logits_idx
            x = x.index_select(0, idx)
            pending = tuple(a.index_select(0, idx) for a in pending)
        hf = hops.add_norm(x, pending, None, self.final_norm, c.norm_eps, True, self.dtype)
        return F.linear(hf, self.head).float() * c.logit_scale

    def _forward_sequential(self, ids: torch.Tensor, meta: AttnMeta, caches: list) -> torch.Tensor:
        """Pre-norm blocks with two norms.  Without depth average the stream is updated in place and
        a layer's feed-forward output is folded into the next layer's norm launch.  With it, entry
        n + 1 of the stack is layer n's working stream (its input, then += mixer, then += feed-forward
        = the layer's result) and depth_mix leaves the next layer's input in entry n + 2."""
        c = self.cfg
        T, d, L = ids.numel(), c.d_model, len(self.runs)
        seg = (meta.seg_cu, meta.seg_ctx, meta.seg_slot)
        if self.depth_avg:
            stack = torch.empty(L + 2, T, d, dtype=torch.float32, device=self.device)
            hops.embed_pos(ids, meta.positions, self.embed, self.pos, meta.dec_src, meta.dec_prev, out=stack[0])
            stack[1].copy_(stack[0])
            x = stack[1]
        else:
            x = hops.embed_pos(ids, meta.positions, self.embed, self.pos, meta.dec_src, meta.dec_prev)
        pending: tuple = ()
        for r, (li, t, first) in enumerate(self.runs):
            if first and self.loop_step is not None:
                x += self.loop_step[t]
            if self.shifted:
                h = hops.norm_shift(x, pending, self.norms[li], c.norm_eps, self.one_plus, self.shifts[li],
                                    caches[r]["shift"], *seg, self.dtype, multi=meta.is_prefill)
            else:
                h = hops.add_norm(x, pending, None, self.norms[li], c.norm_eps, self.one_plus, self.dtype)
            pending = (self.mixers[li].forward(h, meta, caches[self.kv_run[r]]),)
            ff = self.ffns[li]
            if ff is not None:
                h2 = hops.add_norm(x, pending, None, self.norms2[li], c.norm_eps, self.one_plus, self.dtype)
                pending = (ff.forward(h2),)
            if self.depth_avg:
                x = hops.depth_mix(stack, r + 1, pending[0], self.dwa[li])
                pending = ()
            if self.layer_probe is not None:
                self.layer_probe.append(x + sum(a.float() for a in pending))
        if meta.logits_idx is not None:
            idx = meta.logits_idx
            x = x.index_select(0, idx)
            pending = tuple(a.index_select(0, idx) for a in pending)
        hf = hops.add_norm(x, pending, None, self.final_norm, c.norm_eps, self.one_plus, self.dtype)
        return F.linear(hf, self.head).float() * c.logit_scale


def state_dict(model: HybridLM) -> dict:
    """name -> tensor under the checkpoint's names (exporting a random-init model)."""
    out = {"embed": model.embed, "final.norm": model.final_norm, "head": model.head}
    if model.pos is not None:
        out["pos"] = model.pos
    if model.loop_step is not None:
        out["loop.step"] = model.loop_step
    for i, (n, m, f) in enumerate(zip(model.norms, model.mixers, model.ffns)):
        p = f"l{i}."
        out[p + "norm1"] = n
        for key, t in (("norm2", model.norms2[i]), ("shift", model.shifts[i]), ("dwa", model.dwa[i])):
            if t is not None:
                out[p + key] = t
        if isinstance(m, LatentAttention):
            out.update({p + "mix.dq": m.w_down[:m.Q], p + "mix.dq.norm": m.qn, p + "mix.uq": m.w_uq, p + "mix.uk": m.w_uk,
                        p + "mix.uv": m.w_uv, p + "mix.sink": m.sinks, p + "mix.o": m.wo})
            if m.kv_from is None:
                out.update({p + "mix.dkv": m.w_down[m.Q:], p + "mix.dkv.norm": m.kn})
        elif isinstance(m, WindowAttention):
            nq, nk = m.H * m.dk, m.G * m.dk
            out.update({p + "mix.q": m.wqkv[:nq], p + "mix.k": m.wqkv[nq:nq + nk], p + "mix.v": m.wqkv[nq + nk:],
                        p + "mix.q.norm": m.qn, p + "mix.k.norm": m.kn, p + "mix.o": m.wo})
        else:
            out.update({p + "mix.in": m.w_in, p + "mix.conv": m.conv_w, p + "mix.conv.b": m.conv_b,
                        p + "mix.dt_bias": m.dt_bias, p + "mix.A_log": m.a_log, p + "mix.D": m.d_skip,
                        p + "mix.norm": m.norm_w, p + "mix.o": m.wo})
        if isinstance(f, DenseFFN):
            out.update({p + "mlp.up": f.w_up, p + "mlp.down": f.w_down, p + "mlp.act": f.act})
        elif isinstance(f, PlainRoutedFFN):
            for e in range(f.E):
                out[f"{p}mlp.e{e}.up"], out[f"{p}mlp.e{e}.down"] = f.w1[e], f.w2[e]
            out[p + "mlp.router"] = f.wr
            if f.fs:
                out.update({p + "mlp.shared.up": f.ws1, p + "mlp.shared.down": f.ws2})
        elif f is not None:
            for e in range(f.E):
                w13 = _ops.deinterleave_gate_up(f.w13[e]) if f.il else f.w13[e]
                out[f"{p}mlp.e{e}.gate"], out[f"{p}mlp.e{e}.up"] = w13[:f.ff], w13[f.ff:]
                out[f"{p}mlp.e{e}.down"] = f.w2[e]
            out[p + "mlp.router"], out[p + "mlp.router.b"] = f.wr[:f.E], f.bias
            if f.fs:
                out.update({p + "mlp.shared.gate": f.ws13[:f.fs], p + "mlp.shared.up": f.ws13[f.fs:],
                            p + "mlp.shared.down": f.ws2, p + "mlp.shared.sg": f.wr[f.E:]})
    return {k: v.detach().to("cpu", torch.bfloat16).contiguous() for k, v in out.items()}
