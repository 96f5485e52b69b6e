"""Slow, plain float64 forward of the Dunesun design, written straight from its equations: one
function per mechanism, whole sequences at once, no cache, no state carried between calls, no
kernels and nothing imported from the framework.  The tests compare the engine with it.

``cfg`` is the model's ``config.json`` as a dict and ``w`` a dict name -> tensor with the
checkpoint's names (``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``embed``, ``pos``,
``loop.step``, ``final.norm``, ``head``).
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def _w(w: dict, name: str) -> torch.Tensor:
    return w[name].to(F64)


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * (1.0 + weight)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def attention_window_sink(h: torch.Tensor, w: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    """Grouped-query attention without positions in the scores, a sliding window of
    ``mask.size`` keys (the token itself included) and a softmax whose denominator has one more
    term exp(0) that carries no value."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ _w(w, p + "q").T
    k = h @ _w(w, p + "k").T
    v = h @ _w(w, p + "v").T
    q = unit_rms(q, eps) * _w(w, p + "q.norm")  # over the whole projection, before the head split
    k = unit_rms(k, eps) * _w(w, p + "k.norm")
    q = q.view(T, H, dk)
    k = k.view(T, G, dk)
    v = v.view(T, G, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    win = m["mask"]["size"]
    for i in range(T):
        lo = max(0, i - win + 1)
        for hd in range(H):
            g = hd // (H // G)
            s = (k[lo:i + 1, g] @ q[i, hd]) * m["scale"]
            e = torch.exp(s)
            pr = e / (1.0 + e.sum())
            out[i, hd] = pr @ v[lo:i + 1, g]
    return out.reshape(T, H * dv) @ _w(w, p + "o").T


def mamba2(h: torch.Tensor, w: dict, p: str, m: dict, eps: float) -> torch.Tensor:
    """Selective state space layer, token by token from a zero state."""
    T = h.shape[0]
    nh, P, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = nh * P
    proj = h @ _w(w, p + "in").T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    cw, cb = _w(w, p + "conv"), _w(w, p + "conv.b")
    C = xbc.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=F64), xbc])
    conv = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        # the last column of the filter multiplies the current token
        conv[t] = (padded[t:t + taps] * cw.T).sum(0) + cb
    conv = silu(conv)
    x = conv[:, :inner].view(T, nh, P)
    B = conv[:, inner:inner + G * N].view(T, G, N)
    Cm = conv[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + _w(w, p + "dt_bias"))
    A = torch.exp(_w(w, p + "A_log"))
    D = _w(w, p + "D")
    S = torch.zeros(nh, N, P, dtype=F64)
    y = torch.zeros(T, nh, P, dtype=F64)
    for t in range(T):
        for hd in range(nh):
            g = hd // (nh // G)
            S[hd] = torch.exp(-A[hd] * dt[t, hd]) * S[hd] + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S[hd].T @ Cm[t, g] + D[hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)  # the gate comes before the norm
    ng = m["norm_groups"]
    y = unit_rms(y.view(T, ng, inner // ng), eps).reshape(T, inner) * _w(w, p + "norm")
    return y @ _w(w, p + "o").T


def expert(h: torch.Tensor, w: dict, p: str) -> torch.Tensor:
    return (silu(h @ _w(w, p + "gate").T) * (h @ _w(w, p + "up").T)) @ _w(w, p + "down").T


def moe(h: torch.Tensor, w: dict, p: str, m: dict) -> torch.Tensor:
    """Top-k routed experts (softmax over the chosen logits only) plus a shared expert scaled by
    a per-token sigmoid gate."""
    E, K = m["router"]["experts"], m["router"]["top"]
    logits = h @ _w(w, p + "router").T + _w(w, p + "router.b")
    top, idx = torch.topk(logits, K, dim=-1)
    wt = torch.softmax(top, -1)
    out = torch.zeros(h.shape[0], _w(w, p + "e0.down").shape[0], dtype=F64)
    for e in range(E):
        rows, slot = torch.nonzero(idx == e, as_tuple=True)
        if rows.numel():
            out[rows] += expert(h[rows], w, f"{p}e{e}.") * wt[rows, slot].unsqueeze(-1)
    if m.get("shared") is not None:
        gate = torch.sigmoid(h @ _w(w, p + "shared.sg").T)
        out = out + expert(h, w, p + "shared.") * gate
    return out


MIXERS = {"attention": attention_window_sink, "mamba2": mamba2}


def layer(x: torch.Tensor, w: dict, i: int, spec: dict, eps: float) -> torch.Tensor:
    """Parallel block: one norm feeds the mixer and the feed-forward, both are added."""
    p = f"l{i}."
    h = norm_one_plus(x, _w(w, p + "norm1"), eps)
    y = MIXERS[spec["type"]](h, w, p + "mix.", spec["mixer"], eps)
    if spec.get("mlp") is not None:
        y = y + moe(h, w, p + "mlp.", spec["mlp"])
    return x + y


def layer_runs(cfg: dict) -> list:
    """(layer index, pass number or None, first of its pass) in execution order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, None, False) for i in range(a)]
    for t in range(times):
        runs += [(i, t, i == a) for i in range(a, b)]
    runs += [(i, None, False) for i in range(b, n)]
    return runs


def forward(cfg: dict, w: dict, tokens: list, want_layers: bool = False):
    """Logits [T, vocab] (float64) of one whole sequence; with ``want_layers`` also the residual
    stream after every layer run [runs, T, width]."""
    ids = torch.as_tensor(tokens, dtype=torch.long)
    T = ids.numel()
    eps = cfg["norm"]["eps"]
    x = _w(w, "embed")[ids] + _w(w, "pos")[:T]
    x0 = x.clone()
    outs = []
    for i, t, first in layer_runs(cfg):
        if first:
            if t > 0:
                x = x + x0
            x = x + _w(w, "loop.step")[t]
        x = layer(x, w, i, cfg["layers"][i], eps)
        outs.append(x.clone())
    hfin = norm_one_plus(x, _w(w, "final.norm"), eps)
    logits = hfin @ _w(w, "head").T * cfg.get("logit_scale", 1.0)
    return (logits, torch.stack(outs)) if want_layers else logits


def greedy(cfg: dict, w: dict, prompt: list, n: int) -> list:
    ids = list(prompt)
    out = []
    for _ in range(n):
        t = int(torch.argmax(forward(cfg, w, ids)[-1]))
        out.append(t)
        ids.append(t)
    return out


def random_weights(cfg: dict, seed: int = 0, std: float = 0.05) -> dict:
    """Random bf16 weights with the checkpoint's names and shapes for ``cfg``."""
    g = torch.Generator().manual_seed(seed)

    def r(*shape, s=std, mean=0.0):
        return (torch.randn(*shape, generator=g) * s + mean).to(torch.bfloat16)

    d, V = cfg["width"], cfg["vocab"]
    w = {"embed": r(V, d, s=0.5), "pos": r(cfg["max_positions"], d, s=0.1), "final.norm": r(d, s=0.1),
         "head": r(V, d, s=1.0 / math.sqrt(d))}
    loop = cfg.get("loop")
    if loop:
        w["loop.step"] = r(loop["times"], d, s=0.1)
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        w[p + "norm1"] = r(d, s=0.1)
        if spec["type"] == "attention":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            w[p + "mix.q"] = r(H * dk, d, s=1 / math.sqrt(d))
            w[p + "mix.k"] = r(G * dk, d, s=1 / math.sqrt(d))
            w[p + "mix.v"] = r(G * dv, d, s=1 / math.sqrt(d))
            w[p + "mix.q.norm"] = r(H * dk, s=0.2, mean=1.0)
            w[p + "mix.k.norm"] = r(G * dk, s=0.2, mean=1.0)
            w[p + "mix.o"] = r(d, H * dv, s=1 / math.sqrt(H * dv))
        else:
            nh, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, ch = nh * P, nh * P + 2 * G * N
            w[p + "mix.in"] = r(2 * inner + 2 * G * N + nh, d, s=1 / math.sqrt(d))
            w[p + "mix.conv"] = r(ch, m["conv"], s=0.5)
            w[p + "mix.conv.b"] = r(ch, s=0.1)
            w[p + "mix.dt_bias"] = r(nh, s=0.5, mean=-1.0)
            w[p + "mix.A_log"] = r(nh, s=0.5, mean=-0.5)
            w[p + "mix.D"] = r(nh, s=0.5, mean=1.0)
            w[p + "mix.norm"] = r(inner, s=0.2, mean=1.0)
            w[p + "mix.o"] = r(d, inner, s=1 / math.sqrt(inner))
        ml = spec.get("mlp")
        if ml is not None:
            E, ff = ml["router"]["experts"], ml["expert"]["ff"]
            for e in range(E):
                w[p + f"mlp.e{e}.gate"] = r(ff, d, s=1 / math.sqrt(d))
                w[p + f"mlp.e{e}.up"] = r(ff, d, s=1 / math.sqrt(d))
                w[p + f"mlp.e{e}.down"] = r(d, ff, s=1 / math.sqrt(ff))
            w[p + "mlp.router"] = r(E, d, s=2 / math.sqrt(d))
            w[p + "mlp.router.b"] = r(E, s=0.2)
            if ml.get("shared") is not None:
                fs = ml["shared"]["ff"]
                w[p + "mlp.shared.gate"] = r(fs, d, s=1 / math.sqrt(d))
                w[p + "mlp.shared.up"] = r(fs, d, s=1 / math.sqrt(d))
                w[p + "mlp.shared.down"] = r(d, fs, s=1 / math.sqrt(fs))
                w[p + "mlp.shared.sg"] = r(1, d, s=1 / math.sqrt(d))
    return w
