"""Slow, plain float64 forward of the Kisutar design, written from its equations: one function
per mechanism, whole sequences at once, keys and values of every head written out (no latent
cache, no absorbed products), no state carried between calls, no kernels and nothing imported
from the framework.  The tests compare the engine with it.

``cfg`` is the model's ``config.json`` as a dict and ``w`` a dict name -> tensor with the
checkpoint's names (``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.shift``, ``l<i>.dwa``,
``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``).
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def _w(w: dict, name: str) -> torch.Tensor:
    return w[name].to(F64)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def token_shift(h: torch.Tensor, mu: torch.Tensor) -> torch.Tensor:
    """Row t moves towards row t - 1 (as it was before any moving; zeros before the first row) by
    the per-channel fraction ``mu``."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]])
    return h + (prev - h) * mu


def rotate(v: torch.Tensor, pos: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """v [T, ..., n]: the first ``dims`` entries of the last axis are turned in pairs (i, i + dims/2)
    by the angle pos * base^(-2i/dims); the rest pass."""
    half = dims // 2
    out = v.clone()
    shape = [v.shape[0]] + [1] * (v.dim() - 1)
    for i in range(half):
        a = pos.to(F64) * base ** (-2.0 * i / dims)
        c, s = torch.cos(a).view(shape)[..., 0], torch.sin(a).view(shape)[..., 0]
        u, x = v[..., i], v[..., i + half]
        out[..., i] = u * c - x * s
        out[..., i + half] = x * c + u * s
    return out


def latent_kv(h: torch.Tensor, w: dict, p: str, m: dict, eps: float):
    """The compressed key/value stream of a layer that has its own down-projection: the normed
    latent [T, kv_rank] and the one rotated key part shared by all heads [T, rot_dim]."""
    T = h.shape[0]
    R = m["kv_rank"]
    d = h @ _w(w, p + "dkv").T
    c = rms_norm(d[:, :R], _w(w, p + "dkv.norm"), eps)
    kr = rotate(d[:, R:], torch.arange(T), m["rot"]["base"], m["rot"]["dims"])
    return c, kr


def latent_attention(h: torch.Tensor, w: dict, p: str, m: dict, eps: float, c: torch.Tensor, kr: torch.Tensor):
    """Attention whose queries go through a low-rank bottleneck and whose keys and values are
    expanded per head from the latent ``c``; every head's key also carries ``kr``.  Sliding window
    of ``mask.size`` keys (the token itself included); the softmax denominator has one more term
    exp(sink_h) per head that carries no value."""
    T = h.shape[0]
    H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    cq = rms_norm(h @ _w(w, p + "dq").T, _w(w, p + "dq.norm"), eps)
    q = (cq @ _w(w, p + "uq").T).view(T, H, dn + dr)
    qn = q[..., :dn]
    qr = rotate(q[..., dn:], torch.arange(T), m["rot"]["base"], m["rot"]["dims"])
    kn = (c @ _w(w, p + "uk").T).view(T, H, dn)
    v = (c @ _w(w, p + "uv").T).view(T, H, dv)
    sink = _w(w, p + "sink")
    win = int(m["mask"]["size"])
    out = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        lo = max(0, i - win + 1)
        for hd in range(H):
            s = (kn[lo:i + 1, hd] @ qn[i, hd] + kr[lo:i + 1] @ qr[i, hd]) * m["scale"]
            e = torch.exp(s)
            out[i, hd] = (e / (e.sum() + torch.exp(sink[hd]))) @ v[lo:i + 1, hd]
    return out.reshape(T, H * dv) @ _w(w, p + "o").T


def xielu(z: torch.Tensor, p: torch.Tensor, q: torch.Tensor) -> torch.Tensor:
    pos = softplus(p) * z * z + 0.5 * z
    neg = (0.5 + softplus(q)) * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def dense_ff(h: torch.Tensor, w: dict, p: str) -> torch.Tensor:
    a = _w(w, p + "act")
    return xielu(h @ _w(w, p + "up").T, a[0], a[1]) @ _w(w, p + "down").T


def plain_expert(h: torch.Tensor, w: dict, p: str) -> torch.Tensor:
    return gelu_erf(h @ _w(w, p + "up").T) @ _w(w, p + "down").T


def routed_ff(h: torch.Tensor, w: dict, p: str, ml: dict) -> torch.Tensor:
    """Softmax over ALL experts' logits; the ``top`` largest are used with their probabilities as
    they are (they do not sum to one); a shared expert, if any, is added for every token."""
    E, K = ml["router"]["experts"], ml["router"]["top"]
    s = torch.softmax(h @ _w(w, p + "router").T, -1)
    out = torch.zeros(h.shape[0], _w(w, p + "e0.down").shape[0], dtype=F64)
    for t in range(h.shape[0]):
        chosen = sorted(range(E), key=lambda e: (-float(s[t, e]), e))[:K]
        for e in chosen:
            out[t] += s[t, e] * plain_expert(h[t:t + 1], w, f"{p}e{e}.")[0]
    if ml.get("shared"):
        out += plain_expert(h, w, p + "shared.")
    return out


def forward(cfg: dict, w: dict, tokens, return_layers: bool = False):
    """Logits [T, vocab] of one sequence from position 0 (and the stream after every layer)."""
    eps = cfg["norm"]["eps"]
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x = _w(w, "embed")[ids]
    results = [x]  # X_0 = the embedding output, X_(i+1) = layer i's result before averaging
    kv: dict = {}
    layers = []
    for i, spec in enumerate(cfg["layers"]):
        L = f"l{i}."
        m = spec["mixer"]
        assert spec["type"] == "latent_attention"
        h = token_shift(rms_norm(x, _w(w, L + "norm1"), eps), _w(w, L + "shift"))
        src = m.get("kv_from")
        if src is None:
            kv[i] = latent_kv(h, w, L + "mix.", m, eps)
            src = i
        x = x + latent_attention(h, w, L + "mix.", m, eps, *kv[src])
        ml = spec.get("mlp")
        if ml is not None:
            h2 = rms_norm(x, _w(w, L + "norm2"), eps)
            x = x + (dense_ff(h2, w, L + "mlp.") if ml["kind"] == "dense" else routed_ff(h2, w, L + "mlp.", ml))
        results.append(x)
        a = _w(w, L + "dwa")
        x = sum(a[j] * results[j] for j in range(i + 2))
        layers.append(x)
    logits = rms_norm(x, _w(w, "final.norm"), eps) @ _w(w, "head").T
    return (logits, torch.stack(layers)) if return_layers else logits


def random_weights(cfg: dict, seed: int = 0) -> dict:
    """Random tensors of a config's shapes (values a bf16 checkpoint could hold), by name."""
    g = torch.Generator().manual_seed(seed)
    d, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16).float()

    w = {"embed": rnd(V, d, std=0.7), "final.norm": rnd(d, std=0.1, mean=1.0), "head": rnd(V, d, std=d ** -0.5)}
    for i, spec in enumerate(cfg["layers"]):
        L, m = f"l{i}.", spec["mixer"]
        H, dn, dr, dv, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        w[L + "norm1"] = rnd(d, std=0.1, mean=1.0)
        w[L + "shift"] = rnd(d, std=0.25, mean=0.4)
        w[L + "dwa"] = rnd(i + 2, std=0.15, mean=1.0 / (i + 2))
        w[L + "dwa"][i + 1] += 0.5
        P = L + "mix."
        w[P + "dq"], w[P + "dq.norm"] = rnd(Q, d, std=d ** -0.5), rnd(Q, std=0.1, mean=1.0)
        w[P + "uq"] = rnd(H * (dn + dr), Q, std=1.5 * Q ** -0.5)
        if m.get("kv_from") is None:
            w[P + "dkv"], w[P + "dkv.norm"] = rnd(R + dr, d, std=d ** -0.5), rnd(R, std=0.1, mean=1.0)
        w[P + "uk"] = rnd(H * dn, R, std=1.5 * R ** -0.5)
        w[P + "uv"] = rnd(H * dv, R, std=R ** -0.5)
        w[P + "sink"] = rnd(H, std=1.0)
        w[P + "o"] = rnd(d, H * dv, std=(H * dv) ** -0.5)
        ml = spec.get("mlp")
        if ml is None:
            continue
        w[L + "norm2"] = rnd(d, std=0.1, mean=1.0)
        P = L + "mlp."
        if ml["kind"] == "dense":
            f = ml["ff"]
            w[P + "up"], w[P + "down"], w[P + "act"] = rnd(f, d, std=d ** -0.5), rnd(d, f, std=f ** -0.5), rnd(2, std=0.5)
        else:
            f = ml["expert"]["ff"]
            for e in range(ml["router"]["experts"]):
                w[f"{P}e{e}.up"], w[f"{P}e{e}.down"] = rnd(f, d, std=d ** -0.5), rnd(d, f, std=2 * f ** -0.5)
            w[P + "router"] = rnd(ml["router"]["experts"], d, std=2 * d ** -0.5)
            if ml.get("shared"):
                fs = ml["shared"]["ff"]
                w[P + "shared.up"], w[P + "shared.down"] = rnd(fs, d, std=d ** -0.5), rnd(d, fs, std=fs ** -0.5)
    return w


def greedy(cfg: dict, w: dict, prompt, n: int) -> list:
    """``n`` tokens by repeated whole-sequence forwards, each the argmax of the last logits."""
    seq, out = list(prompt), []
    for _ in range(n):
        t = int(torch.argmax(forward(cfg, w, seq)[-1]))
        out.append(t)
        seq.append(t)
    return out
