"""The Dunesun layer-list design in the engine against the plain float64 oracle
(tests/hybrid_oracle.py): each mechanism alone, prefill against token-by-token decoding, prompt
portions down to two tokens, unequal batches, pages and state slots that are reused, window and
page edges, the first tokens, long decoding, odd sizes, and greedy generation through the engine.

Runs on the CPU (the ops' torch forms); the ``gpu`` tests at the end run the same comparisons
through the HIP kernels."""
import json
import math
import os
import subprocess
import sys

import pytest
import torch

import hybrid_oracle as O
from k8s_llm_monitor_amd.engine import EngineConfig, LLMEngine, SamplingParams
from k8s_llm_monitor_amd.engine.block_manager import BlockManager
from k8s_llm_monitor_amd.engine.runner import ModelRunner, RunnerConfig
from k8s_llm_monitor_amd.engine.sequence import Sequence
from k8s_llm_monitor_amd.models.config import get_config, hybrid_config_from_dict, hybrid_config_to_dict
from k8s_llm_monitor_amd.models.hybrid import HybridLM, state_dict
from k8s_llm_monitor_amd.models.registry import build_model, config_from_dir

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ------------------------------------------------------------------ small configurations

def attn(heads=4, kv=2, dim=16, vdim=24, window=6, scale=0.3):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim,
                                           "mask": {"size": window}, "scale": scale}, "mlp": None}


def ssm(heads=4, vdim=8, state=12, groups=2, conv=3, norm_groups=2):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}, "mlp": None}


def moe(experts=5, top=2, ff=20, shared=28):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top},
            "shared": {"ff": shared} if shared else None}


def with_mlp(layer, m):
    return dict(layer, mlp=m)


def make_cfg(layers, width=40, vocab=61, loop=None, logit_scale=1.0, max_positions=512, eps=1e-5):
    c = {"architecture": "Dunesun", "vocab": vocab, "width": width, "layers": layers, "max_positions": max_positions,
         "norm": {"eps": eps}, "logit_scale": logit_scale}
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


FULL = make_cfg([with_mlp(ssm(), moe()), with_mlp(attn(), moe(4, 1, 12, 0)), ssm(2, 20, 9, 1, 4, 1),
                 with_mlp(attn(3, 3, 8, 8, 17, 0.25), moe(7, 3, 8, 16))], loop=(1, 3, 2), logit_scale=1.7)


class Rig:
    """A model + runner + block manager driven step by step, as the trace replayer drives them."""

    def __init__(self, cfg, w=None, seed=0, device="cpu", dtype=torch.float32, num_blocks=64, max_seqs=4):
        self.cfg = cfg
        self.w = w if w is not None else O.random_weights(cfg, seed)
        hc = hybrid_config_from_dict(cfg, "t")

        class Src:  # the checkpoint reader's interface over a dict
            def __init__(s, d):
                s.d = d

            def get(s, k):
                return s.d[k]

            def keys(s):
                return list(s.d)

        self.model = HybridLM(hc, device=device, dtype=dtype, weights=Src(self.w))
        assert not self.model.unused
        self.runner = ModelRunner(self.model, RunnerConfig(max_num_seqs=max_seqs, max_model_len=cfg["max_positions"],
                                                           num_blocks=num_blocks, use_graphs=False, keep_logits=True))
        self.blocks = BlockManager(num_blocks, prefix_caching=False, state_slots=self.runner.num_state_slots)
        self.live = {}

    def step(self, entries, end=()):
        """entries: [(name, tokens)] -> {name: logits [len(tokens), vocab]} (all places wanted)."""
        chunks, decode = [], []
        for name, toks in entries:
            q = self.live.get(name)
            if q is None:
                q = self.live[name] = Sequence(prompt_ids=[], params=SamplingParams(temperature=0.0))
                assert self.blocks.admit(q)
            have = q.num_tokens
            assert self.blocks.ensure_tokens(q, have + len(toks))
            q.prompt_ids.extend(toks)
            q.num_computed = have
            if len(toks) == 1 and have > 0:
                decode.append((name, q))
            else:
                q.chunk = len(toks)
                chunks.append((name, q))
        out = {}
        with torch.no_grad():
            if chunks:
                rows = decode + chunks
                want = [[0]] * len(decode) + [list(range(q.chunk)) for _, q in chunks]
                lg = self.runner.prefill_launch([q for _, q in chunks], [q for _, q in decode], logit_rows=want).logits
                o = 0
                for (name, _), ws in zip(rows, want):
                    out[name] = lg[o:o + len(ws)].float().cpu()
                    o += len(ws)
            elif decode:
                self.runner.decode_collect(self.runner.decode_launch([q for _, q in decode]))
                for i, (name, _) in enumerate(decode):
                    out[name] = self.runner.last_logits[i:i + 1].float().cpu().clone()
        for _, q in chunks:
            q.num_computed += q.chunk
            q.chunk = 0
        for name in end:
            self.blocks.free(self.live.pop(name))
        return out

    def run_cut(self, name, tokens, cuts, end=True):
        """Feed ``tokens`` in portions of the given sizes (the rest one by one); logits of every place."""
        outs, i = [], 0
        sizes = list(cuts) + [1] * len(tokens)
        for n in sizes:
            if i >= len(tokens):
                break
            outs.append(self.step([(name, tokens[i:i + n])])[name])
            i += n
        if end:
            self.blocks.free(self.live.pop(name))
        return torch.cat(outs)


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def close(got, want, tol=2e-4):
    scale = float(want.abs().max())
    err = float((got.double() - want).abs().max())
    assert err <= tol * max(scale, 1.0), f"max abs err {err:.3e} at scale {scale:.3f}"


def close_most(got, want, tol, frac=0.9):
    """bf16 runs: a router decision that is a near tie in fp32 may fall the other way, which moves
    that row (and what follows it in a recurrent state) by far more than rounding.  Such rows are
    few; a wrong window, state or page would move most rows."""
    scale = float(want.pow(2).mean().sqrt())
    err = (got.double() - want).pow(2).mean(-1).sqrt() / scale
    ok = float((err <= tol).double().mean())
    assert ok >= frac, f"only {ok:.2f} of the rows within {tol} (median {float(err.median()):.3e})"


# ------------------------------------------------------------------ mechanisms alone

@pytest.mark.parametrize("layers", [
    [attn()], [attn(2, 1, 8, 8, 1, 1.0)], [attn(4, 4, 12, 20, 100, 0.2)], [ssm()], [ssm(1, 8, 1, 1, 1, 1)],
    [ssm(6, 4, 33, 3, 5, 3)], [with_mlp(attn(), moe())], [with_mlp(ssm(), moe(3, 3, 8, 0))],
    [with_mlp(attn(), moe(9, 1, 4, 4))]], ids=["attn", "attn-w1-mqa", "attn-wide-window", "ssm", "ssm-ones",
                                               "ssm-odd", "moe-shared", "moe-all-experts", "moe-top1"])
def test_single_mechanism_whole_prompt(layers):
    cfg = make_cfg(layers)
    rig = Rig(cfg, seed=3)
    t = toks(45, cfg["vocab"], 1)
    close(rig.run_cut("a", t, [45]), O.forward(cfg, rig.w, t))


def test_loop_passes_and_logit_scale():
    for loop in ((0, 2, 3), (1, 2, 2), (0, 1, 1), None):
        cfg = make_cfg([attn(), with_mlp(ssm(), moe())], loop=loop, logit_scale=0.5)
        rig = Rig(cfg, seed=4)
        t = toks(30, cfg["vocab"], 2)
        close(rig.run_cut("a", t, [30]), O.forward(cfg, rig.w, t))


def test_layer_outputs_match_oracle():
    rig = Rig(FULL, seed=5)
    t = toks(19, FULL["vocab"], 3)
    rig.model.layer_probe = []
    rig.run_cut("a", t, [19])
    _, layers = O.forward(FULL, rig.w, t, want_layers=True)
    assert len(rig.model.layer_probe) == layers.shape[0] == 6
    for got, want in zip(rig.model.layer_probe, layers):
        close(got, want)
    rig.model.layer_probe = None


# ------------------------------------------------------------------ cuts, decoding, batches

def test_prefill_equals_token_by_token_and_portions():
    rig = Rig(FULL, seed=6)
    t = toks(70, FULL["vocab"], 4)
    want = O.forward(FULL, rig.w, t)
    for cuts in ([70], [], [2, 2, 3, 16, 1, 31], [15, 17, 16, 2], [33, 2, 2, 2], [64]):
        close(rig.run_cut("a", t, cuts), want)


def test_first_tokens_and_single_token_prompt():
    rig = Rig(FULL, seed=7)
    for n in (1, 2, 3):
        t = toks(n, FULL["vocab"], 10 + n)
        close(rig.run_cut("a", t, [n]), O.forward(FULL, rig.w, t))
        close(rig.run_cut("a", t, []), O.forward(FULL, rig.w, t))


def test_long_decoding_past_windows_and_pages():
    rig = Rig(FULL, seed=8)
    t = toks(150, FULL["vocab"], 5)
    close(rig.run_cut("a", t, [20]), O.forward(FULL, rig.w, t))  # 130 decode steps over 9 pages


def test_unequal_batch_equals_each_alone_and_reuse():
    """Four live requests with portions beside decode tokens; one ends and its pages and slot are
    taken by a new request whose logits must not see the old state."""
    rig = Rig(FULL, seed=9, num_blocks=24)
    V = FULL["vocab"]
    T = {n: toks(k, V, s) for n, k, s in (("a", 50, 1), ("b", 21, 2), ("c", 3, 3), ("d", 37, 4), ("e", 44, 5))}
    want = {n: O.forward(FULL, rig.w, t) for n, t in T.items()}
    got = {n: [] for n in T}
    at = {n: 0 for n in T}

    def go(plan, end=()):
        entries = []
        for n, k in plan:
            entries.append((n, T[n][at[n]:at[n] + k]))
            at[n] += k
        for n, lg in rig.step(entries, end).items():
            got[n].append(lg)

    go([("a", 17), ("b", 2), ("c", 3)], end=["c"])
    go([("a", 1), ("b", 19), ("d", 30)], end=["b"])
    slot_b = None
    go([("a", 1), ("d", 1), ("e", 16)])  # e takes the freed slot and pages
    go([("a", 31), ("d", 2), ("e", 1)], end=["a"])
    go([("d", 1), ("e", 1)])
    go([("d", 3), ("e", 26)], end=["d", "e"])
    assert slot_b is None and not rig.live
    for n in T:
        assert at[n] == len(T[n])
        close(torch.cat(got[n]), want[n])
    assert rig.blocks.num_free == 24 and len(rig.blocks._free_slots) == 4


# ------------------------------------------------------------------ edges made visible

def _spiked(cfg, seed, layer, far_pos, n, kind):
    """Weights and a prompt in which ONE far position dominates: its token gets a huge key / value
    (attention) so a window off by one changes the logits far beyond rounding."""
    w = O.random_weights(cfg, seed)
    t = toks(n, cfg["vocab"] - 1, seed)
    special = cfg["vocab"] - 1
    t[far_pos] = special
    w["embed"] = w["embed"].clone()
    w["embed"][special] *= 6.0
    if kind == "attention":
        w[f"l{layer}.mix.v"] = w[f"l{layer}.mix.v"] * 4.0
    return w, t


@pytest.mark.parametrize("win", [1, 2, 5, 16, 17, 33])
def test_window_edge_in_and_out(win):
    """The query at distance win-1 from the spiked key sees it, at distance win it does not; in a
    whole prompt, in decoding, and with the key on the page before."""
    cfg = make_cfg([attn(2, 1, 8, 8, win, 0.5)], width=24, vocab=37)
    far = 30
    w, t = _spiked(cfg, 11, 0, far, far + win + 4, "attention")
    want = O.forward(cfg, w, t)
    inside, outside = want[far + win - 1], want[far + win]
    # the oracle itself distinguishes the two sides clearly (otherwise the test shows nothing)
    t2 = list(t)
    t2[far] = 0
    moved = O.forward(cfg, w, t2)
    assert float((moved[far + win - 1] - inside).abs().max()) > 1e-2
    assert float((moved[far + win] - outside).abs().max()) < 1e-9
    for cuts in ([len(t)], [far + 1], [far - 3, 7], [2] * ((far + win) // 2)):
        rig = Rig(cfg, w=w)
        close(rig.run_cut("a", t, cuts), want, tol=1e-4)


def test_far_state_survives_hundreds_of_tokens():
    """A recurrent layer with slow decay carries one early token to the end."""
    cfg = make_cfg([ssm(2, 8, 6, 1, 2, 1)], width=24, vocab=37)
    w, t = _spiked(cfg, 12, 0, 3, 300, "mamba2")
    w["l0.mix.A_log"] = torch.full_like(w["l0.mix.A_log"], -6.0)  # decay exp(-exp(-6) dt): near 1
    want = O.forward(cfg, w, t)
    t2 = list(t)
    t2[3] = 0
    assert float((O.forward(cfg, w, t2)[-1] - want[-1]).abs().max()) > 1e-3
    for cuts in ([300], [130, 2, 64], [5]):
        close(Rig(cfg, w=w).run_cut("a", t, cuts), want, tol=1e-4)


def test_sink_matters():
    """Leaving the sink term out would change the logits: the kernel's result is the oracle's."""
    cfg = make_cfg([attn(2, 2, 8, 8, 4, 0.05)], width=24, vocab=37)  # small scores: the sink weighs ~1/(n+1)
    rig = Rig(cfg, seed=13)
    t = toks(12, 37, 6)
    close(rig.run_cut("a", t, [12]), O.forward(cfg, rig.w, t), tol=1e-4)


# ------------------------------------------------------------------ engine entry points

def _save(tmp_path, cfg, w):
    from safetensors.torch import save_file

    d = tmp_path / "m"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in w.items()}, str(d / "model.safetensors"))
    return d


def test_greedy_generation_through_engine(tmp_path):
    w = O.random_weights(FULL, 21)
    d = _save(tmp_path, FULL, w)
    assert config_from_dir(d).arch == "dunesun"
    eng = LLMEngine(EngineConfig(model=str(d), weights=str(d), max_num_seqs=3, max_model_len=256, num_blocks=40,
                                 dtype="float32", max_prefill_tokens=16, mixed_prefill_tokens=8), device="cpu")
    prompts = [toks(n, FULL["vocab"], 30 + n) for n in (4, 29, 18, 40)]  # 4 requests over 3 slots: one waits
    seqs = eng.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True))
    for p, s in zip(prompts, seqs):
        assert s.output_ids == O.greedy(FULL, w, p, 10)
    st = eng.stats()
    assert st["mixed_steps"] > 0 and st["kv_blocks_free"] == st["kv_blocks_total"]


def test_preset_round_trip_and_registry():
    c = get_config("dunesun-tiny")
    assert hybrid_config_from_dict(hybrid_config_to_dict(c), c.name) == c
    m = build_model(c, device="cpu", dtype=torch.float32)
    w = state_dict(m)
    cfg = hybrid_config_to_dict(c)
    eng_cfg = EngineConfig(model="dunesun-tiny", max_num_seqs=2, max_model_len=128, num_blocks=16, dtype="float32")
    eng = LLMEngine(eng_cfg, device="cpu")
    p = toks(11, c.vocab_size, 1)
    s = eng.generate([p], SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True))[0]
    assert s.output_ids == O.greedy(cfg, w, p, 6)


def test_state_slots_in_block_manager():
    bm = BlockManager(8, prefix_caching=True, state_slots=2)
    assert not bm.prefix_caching  # a recurrent state cannot be rebuilt from cached prefix pages
    a, b, c = (Sequence(prompt_ids=[1] * 20, params=SamplingParams()) for _ in range(3))
    assert bm.allocate(a) and bm.allocate(b) and {a.state_slot, b.state_slot} == {0, 1}
    assert not bm.can_allocate(c) and not bm.allocate(c) and c.state_slot == -1
    bm.free(a)
    assert bm.allocate(c) and c.state_slot == 0 and a.state_slot == -1


def test_trace_command_replays_steps(tmp_path):
    """The command-line replayer: portions, a mixed step, a decode-only step, ends and reuse."""
    w = O.random_weights(FULL, 22)
    d = _save(tmp_path, FULL, w)
    V = FULL["vocab"]
    A, B = toks(23, V, 1), toks(9, V, 2)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": A[:20], "want": [0, 19]}], "end": []},
             {"step": 1, "entries": [{"id": "y", "tokens": B[:8], "want": [7]}, {"id": "x", "tokens": A[20:21], "want": [0]}],
              "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": A[21:22], "want": []}, {"id": "y", "tokens": B[8:], "want": [0]}],
              "end": ["y"]},
             {"step": 3, "entries": [{"id": "x", "tokens": A[22:], "want": [0]}], "end": ["x"]}]
    out = tmp_path / "o"
    r = subprocess.run([sys.executable, "-m", "k8s_llm_monitor_amd.cmd.trace_run", "--model", str(d), "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "64", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(4)]
    wa, wb = O.forward(FULL, w, A), O.forward(FULL, w, B)
    import numpy as np

    def rd(i):
        return torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V).copy())

    close(rd(0), wa[[0, 19]])
    close(rd(1), torch.stack([wb[7], wa[20]]))  # entry order, not the engine's row order
    close(rd(2), wb[8:9])
    close(rd(3), wa[22:23])


# ------------------------------------------------------------------ the same through the HIP kernels

@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpu_cuts_and_batches_match_oracle(dtype):
    cmp = close if dtype == torch.float32 else (lambda g, w: close_most(g, w, 0.05))
    rig = Rig(FULL, seed=6, device="cuda", dtype=dtype)
    t = toks(70, FULL["vocab"], 4)
    want = O.forward(FULL, rig.w, t)
    for cuts in ([70], [2, 2, 3, 16, 1, 31], [33, 2, 2, 2]):
        cmp(rig.run_cut("a", t, cuts), want)
    u = toks(40, FULL["vocab"], 8)
    wu = O.forward(FULL, rig.w, u)
    a = rig.step([("a", t[:30]), ("b", u[:5])])
    b = rig.step([("a", t[30:31]), ("b", u[5:])], end=["b"])
    c = rig.step([("a", t[31:])], end=["a"])
    cmp(torch.cat([a["a"], b["a"], c["a"]]), want)
    cmp(torch.cat([a["b"], b["b"]]), wu)


@pytest.mark.gpu
def test_gpu_bf16_no_experts_is_within_rounding():
    """Without routed experts nothing is discrete: bf16 stays close on every row."""
    cfg = make_cfg([ssm(), attn(), ssm(2, 20, 9, 1, 4, 1), attn(3, 3, 8, 8, 17, 0.25)], loop=(1, 3, 2))
    rig = Rig(cfg, seed=6, device="cuda", dtype=torch.bfloat16)
    t = toks(70, cfg["vocab"], 4)
    want = O.forward(cfg, rig.w, t)
    for cuts in ([70], [2, 2, 3, 16, 1, 31]):
        close_most(rig.run_cut("a", t, cuts), want, 0.05, frac=1.0)


@pytest.mark.gpu
def test_gpu_matrix_core_paths_in_model():
    """Head sizes and expert shapes that take the matrix-core kernels (MFMA prefill attention,
    vector decode attention, MFMA / tile grouped expert GEMMs, the prompt mapping of the scan): every
    cut of a prompt agrees with the oracle, and no worse than the any-size kernels do."""
    cfg = make_cfg([with_mlp(attn(4, 2, 64, 64, 20, 0.125), moe(4, 2, 128, 128)), ssm(4, 32, 16, 2, 4, 2),
                    with_mlp(attn(2, 1, 128, 128, 33, 0.09), None)], width=128, vocab=97, loop=(0, 2, 2),
                   max_positions=640)
    t = toks(600, cfg["vocab"], 4)  # 1200 routed rows in the whole-prompt step: the tile GEMM
    w = O.random_weights(cfg, 6)
    want = O.forward(cfg, w, t)
    scale = float(want.pow(2).mean().sqrt())

    def rms(got):
        return float((got.double() - want).pow(2).mean().sqrt()) / scale

    errs = {}
    for fast in (1, 0):
        rig = Rig(cfg, w=w, device="cuda", dtype=torch.bfloat16, num_blocks=80)
        assert rig.model.uses_tile_gemm
        for m in rig.model.mixers:
            m.fast = fast
        for name, cuts in (("whole", [600]), ("cut", [100, 37, 2, 300, 64]), ("decode", [560])):
            got = rig.run_cut("a", t, cuts)
            close_most(got, want, 0.06)
            errs[(fast, name)] = rms(got)
    for name in ("whole", "cut", "decode"):
        assert errs[(1, name)] <= 1.5 * errs[(0, name)] + 0.005, errs


@pytest.mark.gpu
def test_gpu_greedy_generation_with_graphs():
    eng = LLMEngine(EngineConfig(model="dunesun-tiny", max_num_seqs=4, max_model_len=256, num_blocks=64,
                                 dtype="float32", max_prefill_tokens=32, mixed_prefill_tokens=16), device="cuda")
    eng.warmup()  # decode steps replay from captured hipGraphs
    cfg, w = hybrid_config_to_dict(eng.model_cfg), state_dict(eng.model)
    prompts = [toks(n, 500, 40 + n) for n in (5, 37, 21)]
    seqs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    assert eng.stats()["graph_buckets"]
    for p, s in zip(prompts, seqs):
        assert s.output_ids == O.greedy(cfg, w, p, 12)
