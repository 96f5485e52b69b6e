"""Layer-list decoders: every layer names its token mixer (windowed attention with a softmax
sink, or the Mamba-2 recurrence) and an optional routed feed-forward; a span of layers may run
several times with shared weights.  ``Dunesun`` is the design served so far; its mixers and
feed-forward are registered by name (``MIXERS``) with their sizes and constants read from the
layer's spec, so another layer-list design can reuse them in another order.

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
from .config import HybridConfig, LayerSpec, MoESpec
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


MIXERS = {WindowAttention.kind: WindowAttention, Mamba2Mixer.kind: Mamba2Mixer}


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
        self.embed = p.get("embed", (V, d), 0.5)
        self.pos = p.get("pos", (cfg.max_position, d), 0.1)
        self.loop_step = p.get("loop.step", (cfg.loop[2], d), 0.1, small=True) if cfg.loop else None
        self.norms, self.mixers, self.ffns = [], [], []
        for i, spec in enumerate(cfg.layers):
            if spec.kind not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer {spec.kind!r} (known: {sorted(MIXERS)})")
            self.norms.append(p.get(f"l{i}.norm1", (d,), 0.1, small=True))
            self.mixers.append(MIXERS[spec.kind](spec, d, cfg.norm_eps, p, f"l{i}.mix."))
            self.ffns.append(RoutedFFN(spec.mlp, d, p, f"l{i}.mlp.") if spec.mlp is not None else None)
        self.final_norm = p.get("final.norm", (d,), 0.1, small=True)
        self.head = p.get("head", (V, d), 1.0 / math.sqrt(d))
        self.runs = cfg.runs()
        self.unused = sorted(set(weights.keys()) - p.used) if weights is not None else []
        self.has_state = any(m.kind != "attention" for m in self.mixers)
        # large steps of such layers run on the Mixtral path's tile GEMM (extension _k8sllm_ops)
        self.uses_tile_gemm = any(f is not None and f.il for f in self.ffns)
        self.layer_probe = None  # a list: forward() appends the residual stream after every run

    # ------------------------------------------------------------------ engine interface
    def overlap_ok(self) -> bool:
        return False

    def cache_bytes(self) -> tuple:
        """(bytes per cache page, bytes per state slot) summed over the layer runs."""
        es = torch.empty(0, dtype=self.dtype).element_size()
        per = [self.mixers[i].cache_bytes(es) for i, _, _ in self.runs]
        return sum(a for a, _ in per), sum(b for _, b in per)

    def new_cache(self, num_blocks: int, num_slots: int) -> list:
        """One cache per layer RUN (a looped layer has one per pass)."""
        return [self.mixers[i].new_cache(num_blocks, num_slots, self.dtype, self.device) for i, _, _ in self.runs]

    def resident_weight_bytes(self) -> int:
        n = 0
        for t in self._tensors():
            n += t.numel() * t.element_size()
        return n

    def num_local_params(self) -> int:
        return sum(t.numel() for t in self._tensors())

    def _tensors(self) -> list:
        ts = [self.embed, self.pos, self.final_norm, self.head] + self.norms
        if self.loop_step is not None:
            ts.append(self.loop_step)
        for o in self.mixers + [f for f in self.ffns if f is not None]:
            ts += [v for v in vars(o).values() if isinstance(v, torch.Tensor)]
        return ts

    # ------------------------------------------------------------------ forward
    def forward(self, ids: torch.Tensor, meta: AttnMeta, caches: list) -> torch.Tensor:
        """Logits [rows, vocab] (fp32) for the rows ``meta.logits_idx`` selects (all when None)."""
        c = self.cfg
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


def state_dict(model: HybridLM) -> dict:
    """name -> tensor under the checkpoint's names (exporting a random-init model)."""
    out = {"embed": model.embed, "pos": model.pos, "final.norm": model.final_norm, "head": model.head}
    if model.loop_step is not None:
        out["loop.step"] = model.loop_step
    for i, (n, m, f) in enumerate(zip(model.norms, model.mixers, model.ffns)):
        p = f"l{i}."
        out[p + "norm1"] = n
        if isinstance(m, WindowAttention):
            nq, nk = m.H * m.dk, m.G * m.dk
            out.update({p + "mix.q": m.wqkv[:nq], p + "mix.k": m.wqkv[nq:nq + nk], p + "mix.v": m.wqkv[nq + nk:],
                        p + "mix.q.norm": m.qn, p + "mix.k.norm": m.kn, p + "mix.o": m.wo})
        else:
            out.update({p + "mix.in": m.w_in, p + "mix.conv": m.conv_w, p + "mix.conv.b": m.conv_b,
                        p + "mix.dt_bias": m.dt_bias, p + "mix.A_log": m.a_log, p + "mix.D": m.d_skip,
                        p + "mix.norm": m.norm_w, p + "mix.o": m.wo})
        if f is not None:
            for e in range(f.E):
                w13 = _ops.deinterleave_gate_up(f.w13[e]) if f.il else f.w13[e]
                out[f"{p}mlp.e{e}.gate"], out[f"{p}mlp.e{e}.up"] = w13[:f.ff], w13[f.ff:]
                out[f"{p}mlp.e{e}.down"] = f.w2[e]
            out[p + "mlp.router"], out[p + "mlp.router.b"] = f.wr[:f.E], f.bias
            if f.fs:
                out.update({p + "mlp.shared.gate": f.ws13[:f.fs], p + "mlp.shared.up": f.ws13[f.fs:],
                            p + "mlp.shared.down": f.ws2, p + "mlp.shared.sg": f.wr[f.E:]})
    return {k: v.detach().to("cpu", torch.bfloat16).contiguous() for k, v in out.items()}
