"""Operators of the layer-list (hybrid) decoders: fp32 residual stream with one-plus RMSNorm,
windowed attention with a softmax sink over a paged cache, the Mamba-2 recurrence with its short
convolution and per-sequence state slots, and routed experts with a biased fp32 router and a
gated shared expert.

GPU tensors run the gfx950 kernels of ``_k8sllm_hybrid`` (``ops/csrc/hybrid``; built by
``python -m k8s_llm_monitor_amd.ops.build --only hybrid``) for bfloat16 and float32 activations
alike; CPU tensors run the torch forms below (the same arithmetic in fp32).  A GPU tensor never
falls back: without the extension the call raises.

Conventions.  ``T`` rows are the step's tokens, all sequences concatenated; a *segment* is one
sequence's rows of this step (a decode token is a segment of one row).  ``seg_cu`` [R+1] are the
segments' row offsets, ``seg_ctx`` [R] the tokens each sequence already holds in its cache /
state (0 = the sequence starts here, its state is taken as zero), ``seg_slot`` [R] its state slot
(< 0: a padding row, skipped).  Paged caches: keys ``[blocks, block_size, heads * dim]`` (a token's
keys contiguous), values ``[blocks, heads, vdim, block_size]`` (a value dim's tokens contiguous - the
direction the PV products read along).
"""
from __future__ import annotations

import importlib
from typing import Optional

import torch
import torch.nn.functional as F

_EXT = None
_EXT_ERR: Optional[BaseException] = None


def native():
    """The compiled ``_k8sllm_hybrid`` module (raises with the build hint if unavailable)."""
    global _EXT, _EXT_ERR
    if _EXT is None and _EXT_ERR is None:
        try:
            _EXT = importlib.import_module("k8s_llm_monitor_amd.ops._k8sllm_hybrid")
        except BaseException as e:  # noqa: BLE001 - remembered, re-raised on GPU use
            _EXT_ERR = e
    if _EXT is None:
        raise RuntimeError("gfx950 kernels (_k8sllm_hybrid) are not built/loadable; run "
                           "`python -m k8s_llm_monitor_amd.ops.build --only hybrid` (cause: %r)" % (_EXT_ERR,))
    return _EXT


def native_available() -> bool:
    try:
        native()
        return True
    except RuntimeError:
        return False


def _silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# ---------------------------------------------------------------- residual stream / norms

def embed_pos(ids: torch.Tensor, positions: torch.Tensor, embed: torch.Tensor, pos: Optional[torch.Tensor],
              src: Optional[torch.Tensor] = None, prev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 rows ``embed[id] + pos[position]`` (``pos`` None: no learned positions).  ``src`` /
    ``prev`` (pipelined decode): row i takes token ``prev[src[i]]`` where ``src[i] >= 0``."""
    if not embed.is_cuda:
        if src is not None:
            ids = torch.where(src >= 0, prev.index_select(0, src.clamp(min=0).long()), ids)
        x = embed[ids.long()].float()
        return x + pos[positions.long()].float() if pos is not None else x
    out = torch.empty(ids.numel(), embed.shape[1], dtype=torch.float32, device=embed.device)
    native().embed_pos(out, ids, positions, embed, pos, src, prev)
    return out


def add_norm(residual: torch.Tensor, addends: tuple, vec: Optional[torch.Tensor], w: torch.Tensor, eps: float,
             one_plus: bool, out_dtype: torch.dtype) -> torch.Tensor:
    """``residual`` (fp32 [T, d], updated in place) += sum of ``addends`` ([T, d] each, any float
    dtype, at most three) + ``vec`` ([d], broadcast over the rows); returns the RMSNorm of the new
    residual times ``w`` (``one_plus``: times ``1 + w``) in ``out_dtype``.  The sum and the norm
    are fp32."""
    if not residual.is_cuda:
        for a in addends:
            residual += a.float()
        if vec is not None:
            residual += vec.float()
        y = residual * torch.rsqrt(residual.pow(2).mean(-1, keepdim=True) + eps)
        wf = w.float()
        return (y * (1.0 + wf if one_plus else wf)).to(out_dtype)
    assert len(addends) <= 3
    out = torch.empty(residual.shape, dtype=out_dtype, device=residual.device)
    a = list(addends) + [None] * (3 - len(addends))
    native().add_norm(out, residual, a[0], a[1], a[2], vec, w, float(eps), bool(one_plus))
    return out


# ---------------------------------------------------------------- windowed attention with a sink

def qk_norm_cache(qkv: torch.Tensor, qw: torch.Tensor, kw: torch.Tensor, eps: float, Hq: int, Hkv: int, dk: int,
                  dv: int, k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                  slot_mapping: Optional[torch.Tensor]) -> None:
    """In place on the fused rows [T, Hq*dk | Hkv*dk | Hkv*dv]: q and k are each divided by the
    root mean square of their WHOLE projection (all heads together, fp32) and multiplied by
    ``qw`` / ``kw``; the normed k and v go to the paged cache at ``slot_mapping`` (< 0: not
    written)."""
    nq, nk = Hq * dk, Hkv * dk
    if not qkv.is_cuda:
        q, k = qkv[:, :nq].float(), qkv[:, nq:nq + nk].float()
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * qw.float()
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * kw.float()
        qkv[:, :nq] = q.to(qkv.dtype)
        qkv[:, nq:nq + nk] = k.to(qkv.dtype)
        if k_cache is not None:
            ok = slot_mapping >= 0
            s = slot_mapping[ok].long()
            k_cache.view(-1, nk)[s] = qkv[ok, nq:nq + nk]
            bs = k_cache.shape[1]
            v_cache.view(-1, Hkv * dv, bs)[s // bs, :, s % bs] = qkv[ok, nq + nk:]
        return
    native().qk_norm_cache(qkv, qw, kw, float(eps), Hq, Hkv, dk, dv, k_cache, v_cache, slot_mapping)


def _attend(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, sink: bool) -> torch.Tensor:
    """q [H, dk], k [n, G, dk], v [n, G, dv] (fp32) -> [H, dv]."""
    H, G = q.shape[0], k.shape[1]
    kk = k.repeat_interleave(H // G, dim=1)
    vv = v.repeat_interleave(H // G, dim=1)
    s = torch.einsum("hd,nhd->hn", q, kk) * scale
    m = s.max(-1, keepdim=True).values
    if sink:
        m = m.clamp(min=0.0)
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True) + (torch.exp(-m) if sink else 0.0)
    return torch.einsum("hn,nhd->hd", e / den, vv)


def window_attention_prefill(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, cu: torch.Tensor,
                             ctx: torch.Tensor, block_tables: torch.Tensor, Hq: int, Hkv: int, dk: int, dv: int,
                             scale: float, window: int, sink: bool, mfma: int = 1) -> torch.Tensor:
    """Attention of the step's prompt chunks over the paged cache (which already holds their own
    keys): row r of segment s at position p = ctx[s] + r sees positions max(0, p - window + 1) .. p
    (``window`` 0: all of 0 .. p).  ``sink``: the softmax denominator has one more term exp(0) that
    carries no value.  Scores and weights are fp32.  Returns [T, Hq*dv].  GPU, bf16, head sizes
    64 / 128: the matrix-core kernel, 16 query rows per wave or 32 in large steps (``mfma`` 0: the
    any-size wave-per-row kernel; 16 / 32 / 64: that many rows per wave)."""
    T = qkv.shape[0]
    if not qkv.is_cuda:
        out = torch.empty(T, Hq * dv, dtype=qkv.dtype)
        bs = k_cache.shape[1]
        cul, ctxl = cu.tolist(), ctx.tolist()
        for s in range(len(ctxl)):
            n_all = ctxl[s] + cul[s + 1] - cul[s]
            bt = block_tables[s, : (n_all + bs - 1) // bs].long()
            ks = k_cache[bt].reshape(-1, Hkv, dk)[:n_all].float()
            vs = v_cache[bt].permute(0, 3, 1, 2).reshape(-1, Hkv, dv)[:n_all].float()
            for r in range(cul[s], cul[s + 1]):
                p = ctxl[s] + r - cul[s]
                lo = max(0, p - window + 1) if window > 0 else 0
                o = _attend(qkv[r, : Hq * dk].float().view(Hq, dk), ks[lo:p + 1], vs[lo:p + 1], scale, sink)
                out[r] = o.reshape(-1).to(qkv.dtype)
        return out
    out = torch.empty(T, Hq * dv, dtype=qkv.dtype, device=qkv.device)
    native().window_attention_prefill(out, qkv, k_cache, v_cache, cu, ctx, block_tables, Hq, Hkv, dk, dv, float(scale),
                                      int(window), bool(sink), int(mfma))
    return out


def window_attention_decode(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                            block_tables: torch.Tensor, seq_lens: torch.Tensor, Hq: int, Hkv: int, dk: int, dv: int,
                            scale: float, window: int, sink: bool, vec: bool = True) -> torch.Tensor:
    """One query per sequence (its newest token, already in the cache) over the last ``window``
    cached positions; ``seq_lens`` count that token (0: a padding row, output zero)."""
    B = qkv.shape[0]
    if not qkv.is_cuda:
        out = torch.zeros(B, Hq * dv, dtype=qkv.dtype)
        bs = k_cache.shape[1]
        for b, n in enumerate(seq_lens.tolist()):
            if n <= 0:
                continue
            lo = max(0, n - window) if window > 0 else 0
            bt = block_tables[b, : (n + bs - 1) // bs].long()
            ks = k_cache[bt].reshape(-1, Hkv, dk)[lo:n].float()
            vs = v_cache[bt].permute(0, 3, 1, 2).reshape(-1, Hkv, dv)[lo:n].float()
            out[b] = _attend(qkv[b, : Hq * dk].float().view(Hq, dk), ks, vs, scale, sink).reshape(-1).to(qkv.dtype)
        return out
    out = torch.empty(B, Hq * dv, dtype=qkv.dtype, device=qkv.device)
    native().window_attention_decode(out, qkv, k_cache, v_cache, block_tables, seq_lens, Hq, Hkv, dk, dv, float(scale),
                                     int(window), bool(sink), bool(vec))
    return out


# ---------------------------------------------------------------- Mamba-2

def conv_silu(proj: torch.Tensor, col0: int, C: int, conv_w: torch.Tensor, conv_b: torch.Tensor,
              conv_state: torch.Tensor, seg_cu: torch.Tensor, seg_ctx: torch.Tensor,
              seg_slot: torch.Tensor) -> torch.Tensor:
    """Causal per-channel convolution + SiLU over columns [col0, col0 + C) of ``proj`` [T, *];
    ``conv_w`` [C, taps] (the last tap multiplies the current token), ``conv_b`` [C].  The taps - 1
    inputs before a segment come from ``conv_state`` [slots, taps - 1, C] (zeros where seg_ctx is
    0), which is then advanced to the segment's end."""
    T = proj.shape[0]
    taps = conv_w.shape[1]
    if not proj.is_cuda:
        out = torch.empty(T, C, dtype=proj.dtype)
        wt, bf = conv_w.float().t(), conv_b.float()  # [taps, C]
        cul = seg_cu.tolist()
        for s, (c0, slot) in enumerate(zip(seg_ctx.tolist(), seg_slot.tolist())):
            a, b = cul[s], cul[s + 1]
            if slot < 0 or b <= a:
                continue
            x = proj[a:b, col0:col0 + C]
            hist = conv_state[slot, : taps - 1]
            if c0 <= 0:
                hist = torch.zeros_like(hist)
            full = torch.cat([hist.to(proj.dtype), x]).float()  # [taps - 1 + n, C]
            acc = bf.expand(b - a, C).clone()
            for j in range(taps):
                acc += full[j:j + b - a] * wt[j]
            out[a:b] = _silu(acc).to(proj.dtype)
            if taps > 1:
                conv_state[slot] = full[full.shape[0] - (taps - 1):].to(conv_state.dtype)
        return out
    out = torch.empty(T, C, dtype=proj.dtype, device=proj.device)
    native().conv_silu(out, proj, int(col0), conv_w, conv_b, conv_state, seg_cu, seg_ctx, seg_slot)
    return out


def ssm_scan(xbc: torch.Tensor, proj: torch.Tensor, dt_col: int, dt_bias: torch.Tensor, a_log: torch.Tensor,
             d_skip: torch.Tensor, state: torch.Tensor, seg_cu: torch.Tensor, seg_ctx: torch.Tensor,
             seg_slot: torch.Tensor, nh: int, P: int, N: int, G: int, mode: int = 0) -> torch.Tensor:
    """The selective state-space recurrence, fp32, token by token within each segment:

        dt = softplus(proj[t, dt_col + h] + dt_bias[h]);  S <- exp(-exp(a_log[h]) dt) S + dt B_t x_t^T
        y_t = S^T C_t + d_skip[h] x_t

    ``xbc`` [T, nh*P | G*N | G*N] holds x, B, C (head h reads group h // (nh / G)); ``state``
    [slots, nh, N, P] fp32 is read at the segment's start (zero where seg_ctx is 0) and written
    back at its end.  Returns y [T, nh*P] fp32.  GPU: two lane mappings of the same arithmetic,
    chosen by the step's mean segment length (``mode`` 1 / 2 forces the decode / the prompt one)."""
    T = xbc.shape[0]
    if not xbc.is_cuda:
        y = torch.zeros(T, nh * P, dtype=torch.float32)
        A = torch.exp(a_log.float())
        Dk = d_skip.float()
        cul = seg_cu.tolist()
        inner = nh * P
        for s, (c0, slot) in enumerate(zip(seg_ctx.tolist(), seg_slot.tolist())):
            a, b = cul[s], cul[s + 1]
            if slot < 0 or b <= a:
                continue
            S = state[slot].clone() if c0 > 0 else torch.zeros_like(state[slot])
            xs = xbc[a:b, :inner].float().view(-1, nh, P)
            Bs = xbc[a:b, inner:inner + G * N].float().view(-1, G, N).repeat_interleave(nh // G, dim=1)
            Cs = xbc[a:b, inner + G * N:].float().view(-1, G, N).repeat_interleave(nh // G, dim=1)
            dt = F.softplus(proj[a:b, dt_col:dt_col + nh].float() + dt_bias.float(), threshold=30.0)
            dec = torch.exp(-A * dt)
            for t in range(b - a):
                S = dec[t, :, None, None] * S + dt[t, :, None, None] * Bs[t, :, :, None] * xs[t, :, None, :]
                y[a + t] = (torch.einsum("hnp,hn->hp", S, Cs[t]) + Dk[:, None] * xs[t]).reshape(-1)
            state[slot] = S
        return y
    y = torch.empty(T, nh * P, dtype=torch.float32, device=xbc.device)
    native().ssm_scan(y, xbc, proj, int(dt_col), dt_bias, a_log, d_skip, state, seg_cu, seg_ctx, seg_slot, nh, P, N, G,
                      int(mode))
    return y


def gated_group_norm(y: torch.Tensor, proj: torch.Tensor, z_col: int, w: torch.Tensor, eps: float, groups: int,
                     out_dtype: torch.dtype) -> torch.Tensor:
    """``y`` [T, n] fp32 times silu of the gate ``proj[:, z_col : z_col + n]``, then RMS-normed in
    ``groups`` equal parts (each by its own root mean square) times ``w`` [n]."""
    T, n = y.shape
    if not y.is_cuda:
        g = y * _silu(proj[:, z_col:z_col + n].float())
        g = g.view(T, groups, n // groups)
        g = g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps)
        return (g.reshape(T, n) * w.float()).to(out_dtype)
    out = torch.empty(T, n, dtype=out_dtype, device=y.device)
    native().gated_group_norm(out, y, proj, int(z_col), w, float(eps), int(groups))
    return out


# ---------------------------------------------------------------- routed experts

def moe_router(h: torch.Tensor, wr: torch.Tensor, bias: torch.Tensor, E: int, K: int) -> tuple:
    """fp32 router: logits = ``wr[:E] h + bias[:E]``, the ``K`` largest are chosen and weighted by
    the softmax over the chosen logits only.  ``wr`` may hold one more row (E + 1 in all): then
    ``gate = sigmoid(wr[E] h)`` per token is returned too (the shared expert's gate).
    Returns (ids [T, K] int32, weights [T, K] fp32, gate [T] fp32 or None)."""
    T = h.shape[0]
    has_gate = wr.shape[0] == E + 1
    if not h.is_cuda:
        lg = h.float() @ wr.float().t()
        gate = torch.sigmoid(lg[:, E]) if has_gate else None
        top, idx = torch.topk(lg[:, :E] + bias.float()[:E], K, dim=-1)
        return idx.to(torch.int32), torch.softmax(top, -1), gate
    ids = torch.empty(T, K, dtype=torch.int32, device=h.device)
    wts = torch.empty(T, K, dtype=torch.float32, device=h.device)
    gate = torch.empty(T, dtype=torch.float32, device=h.device) if has_gate else None
    native().moe_router(ids, wts, gate, h, wr, bias, E, K)
    return ids, wts, gate


# expert-sorted rows from which the routed GEMMs of an interleaved (``il``) layer go to the
# framework's 256 x 256 prefill tile kernel (ops.moe_grouped_gemm) instead of the 16-row kernel
TILE_MIN_ROWS = 1024


def moe_experts(h: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor,
                shared: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None, il: bool = False,
                mfma: bool = True) -> torch.Tensor:
    """Sum over each token's chosen experts of ``wts * down_e(silu(gate_e h) * up_e h)`` with
    ``w13`` [E, 2*ff, d] (gate rows then up rows; ``il``: interleaved per 128 rows as [64 gate |
    64 up], ops.interleave_gate_up) and ``w2`` [E, d, ff], plus ``gate * shared`` (the shared
    expert's output [T, d] and its per-token gate).  fp32 [T, d].

    GPU: the (token, slot) pairs are counting-sorted by expert on the device and both projections
    run as ONE grouped launch each over the sorted rows (SwiGLU in the first epilogue); no host
    synchronisation.  bf16: matrix-core kernels - 16-row tiles with the rows gathered on load
    (decode, small steps), or from TILE_MIN_ROWS sorted rows of an ``il`` layer the prefill tile
    GEMM of the Mixtral path; fp32 (and K not a multiple of 32): the 64 x 64 fp32 tile kernel."""
    T, d = h.shape
    E, K = w13.shape[0], ids.shape[1]
    ff = w2.shape[2]
    if not h.is_cuda:
        out = torch.zeros(T, d, dtype=torch.float32)
        hf = h.float()
        for e in range(E):
            rows, slot = torch.nonzero(ids == e, as_tuple=True)
            if rows.numel():
                we = w13[e].float()
                if il:
                    we = we.view(ff // 64, 2, 64, d).permute(1, 0, 2, 3).reshape(2 * ff, d)
                gu = (hf[rows] @ we.t()).to(h.dtype).float()
                act = (_silu(gu[:, :ff]) * gu[:, ff:]).to(h.dtype).float()
                out.index_add_(0, rows, (act @ w2[e].float().t()).to(h.dtype).float() * wts[rows, slot].unsqueeze(-1))
        if shared is not None:
            out += shared.float() * gate.unsqueeze(-1)
        return out
    ext = native()
    n = T * K
    offsets = torch.empty(E + 1, dtype=torch.int32, device=h.device)
    sorted_idx = torch.empty(n, dtype=torch.int32, device=h.device)
    inv_idx = torch.empty(n, dtype=torch.int32, device=h.device)
    ext.moe_align(ids, E, offsets, sorted_idx, inv_idx)
    if il and n >= TILE_MIN_ROWS and h.dtype == torch.bfloat16:
        from .. import ops  # the Mixtral path's kernels (_k8sllm_ops)

        xs = ops.gather_rows(h, sorted_idx, K)
        act = ops.moe_grouped_gemm(xs, w13, offsets, swiglu=True, zero_fill=False)
        ys = ops.moe_grouped_gemm(act, w2, offsets, zero_fill=False)
    else:
        act = torch.empty(n, ff, dtype=h.dtype, device=h.device)
        ext.grouped_gemm(act, h, w13, offsets, sorted_idx, K, True, il, mfma)
        ys = torch.empty(n, d, dtype=h.dtype, device=h.device)
        ext.grouped_gemm(ys, act, w2, offsets, None, 1, False, False, mfma)
    out = torch.empty(T, d, dtype=torch.float32, device=h.device)
    ext.moe_combine(out, ys, inv_idx, wts, shared, gate)
    return out


def swiglu(gu: torch.Tensor) -> torch.Tensor:
    """silu(gu[:, :f]) * gu[:, f:] for [T, 2f] rows ([gate | up])."""
    f = gu.shape[1] // 2
    if not gu.is_cuda:
        return (_silu(gu[:, :f].float()) * gu[:, f:].float()).to(gu.dtype)
    out = torch.empty(gu.shape[0], f, dtype=gu.dtype, device=gu.device)
    native().swiglu(out, gu)
    return out
