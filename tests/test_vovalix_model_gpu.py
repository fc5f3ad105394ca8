"""The Vovalix decoder in the engine against the plain implementation, under every way of
cutting the work: whole prompts, prompts then single tokens, portions down to two tokens,
unequal requests side by side, pages and state slots that are given back and used again, long
decoding, and greedy generation through the engine's own entry point and scheduler."""

from __future__ import annotations

import pytest
import torch

from tests.helpers import random_tokens
from tests.plain import vovalix as plain
from tests.test_cuts_gpu import collect
from tests.vovalix_helpers import CONFIGS, make_model_dir

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, (config, page) in CONFIGS.items():
        folder = make_model_dir(tmp_path_factory.mktemp(f"vovalix_{name}"), config, seed=51 + len(out))
        cfg, weights = plain.load_model_folder(folder)
        out[name] = (folder, cfg, weights, page)
    return out


_oracle: dict = {}
_margins: dict = {}
CLOSE_CALL = 0.15  # of the router logits' spread


def oracle(name, cfg, weights, tokens):
    """The plain model's logits; it also notes how clear the routers' choices were at every
    position (``routing_margin``)."""
    key = (name, tuple(tokens))
    if key not in _oracle:
        margins: list = []
        _oracle[key] = plain.vovalix_forward(cfg, weights, tokens, margins=margins)
        _margins[id(_oracle[key])] = (torch.stack(margins).min(dim=0).values if margins
                                      else torch.full((len(tokens),), float("inf")))
    return _oracle[key]


def routing_margin(logits, pos) -> float:
    m = _margins.get(id(logits))
    return float("inf") if m is None else float(m[pos])


def session_for(folder, dtype, page, max_tokens, **kw):
    from kvcore_amd.engine.replay import TraceSession

    return TraceSession(str(folder), dtype, max_tokens=max_tokens, block_size=page, poison_cache=True, **kw)


def compare(got, expect_by_id, dtype):
    """Logit rows against the plain model's: the difference with its mean taken off, root mean
    square over the vocabulary, relative to the root mean square of the row itself.  float32
    differs by the order of its sums only, and every position must agree (which pins the routing
    itself).  bfloat16 rounds activations to 8 bits at a dozen places a layer, and that can turn a
    router whose two candidates lie close: the token then runs another expert, which is no error
    of the engine.  So in bfloat16 a position may differ by more than the limit only where the
    plain model's own routing was a close call (within ``CLOSE_CALL`` of the logits' spread), at
    most one position in ten; and since the neighbours of such a position read its keys and
    states, one position in fifty may reach one and a half times the limit."""
    limit = 2e-4 if dtype == torch.float32 else 6e-2
    assert got, "nothing was compared"
    worst, excused, over = 0.0, 0, 0
    for (rid, pos), row in sorted(got.items()):
        ref = expect_by_id[rid][pos]
        assert torch.isfinite(row).all(), f"non-finite logits at {rid}:{pos}"
        d = row - ref
        d = d - d.mean()
        err = float(d.pow(2).mean().sqrt() / (ref - ref.mean()).pow(2).mean().sqrt())
        if err <= limit:
            worst = max(worst, err)
        elif dtype == torch.bfloat16 and routing_margin(expect_by_id[rid], pos) < CLOSE_CALL:
            excused += 1
        elif dtype == torch.bfloat16 and err <= 1.5 * limit:
            over += 1
        else:
            raise AssertionError(f"{rid}:{pos} differs by {err:.3e} of its size (limit {limit}; routing margin "
                                 f"{routing_margin(expect_by_id[rid], pos):.3f})")
    assert excused * 10 <= len(got) + 9, f"{excused} of {len(got)} positions differ by a turned router"
    assert over * 50 <= len(got) + 49, f"{over} of {len(got)} positions lie above the limit"
    return worst


def test_the_test_weights_reach_every_expert_and_spread_the_decays(models):
    """What the other tests rest on: the routers send tokens to every expert, and the decays lie
    between fast and slow."""
    folder, cfg, weights, page = models["A"]
    w = {k: v.double() for k, v in weights.items()}
    tokens = random_tokens(75, cfg["vocab"], 5)
    x = plain.offset_rms_norm(w["embed"][torch.tensor(tokens)], w["l0.norm1"], cfg["norm"]["eps"])
    scores = torch.softmax(x @ w["l0.mlp.router"].T, dim=-1)
    seen = set()
    for t in range(len(tokens)):
        seen.update(plain.route(scores[t], 2, 3, 2)[0])
    assert seen == set(range(6))
    decay = torch.sigmoid((x @ w["l1.mix.a1"].T) @ w["l1.mix.a2"].T + w["l1.mix.a2.b"]).pow(1 / 8.0)
    assert float(decay.min()) < 0.9 and float(decay.max()) > 0.99


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompts_then_single_tokens_then_portions(models, name, dtype):
    folder, cfg, weights, page = models[name]
    V = cfg["vocab"]
    tokens = random_tokens(75, V, 5)
    want = {"a": oracle(name, cfg, weights, tokens)}
    s = session_for(folder, dtype, page, 256)
    # whole
    got = collect(s, [{"step": 0, "entries": [{"id": "a", "tokens": tokens, "want": list(range(75))}], "end": ["a"]}])
    compare(got, want, dtype)
    # a prompt, then token by token (the slot and the pages of the first run are used again)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": tokens[:40], "want": [0, 39]}], "end": []}]
    for i in range(40, 75):
        steps.append({"step": i, "entries": [{"id": "a", "tokens": tokens[i: i + 1], "want": [0]}],
                      "end": ["a"] if i == 74 else []})
    compare(collect(s, steps), want, dtype)
    # portions of every size down to two tokens and one, cut inside pages and chunks
    steps, at = [], 0
    for n in (2, 3, 2, 1, 9, 2, 17, 1, 1, 2, 30, 5):
        steps.append({"step": len(steps), "entries": [{"id": "a", "tokens": tokens[at: at + n],
                                                       "want": list(range(n))}],
                      "end": ["a"] if at + n == 75 else []})
        at += n
    assert at == 75
    compare(collect(s, steps), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_unequal_requests_side_by_side_with_slots_used_again(models, name, dtype):
    """Up to three live requests in two slots' worth of pages more than one needs: portions of
    some beside single tokens of others, requests that pause, end and are followed by new ones
    in the same slots and pages (cache and states are poisoned when they are given back)."""
    folder, cfg, weights, page = models[name]
    V = cfg["vocab"]
    seqs = {"a": random_tokens(61, V, 1), "b": random_tokens(33, V, 2), "c": random_tokens(9, V, 3),
            "d": random_tokens(47, V, 4), "e": random_tokens(2, V, 5), "f": random_tokens(1, V, 6)}
    want = {k: oracle(name, cfg, weights, v) for k, v in seqs.items()}
    s = session_for(folder, dtype, page, 192, max_num_seqs=3)
    at = {k: 0 for k in seqs}

    def entry(k, n):
        lo = at[k]
        n = min(n, len(seqs[k]) - lo)
        at[k] += n
        return {"id": k, "tokens": seqs[k][lo: lo + n], "want": list(range(n))}

    plan = [
        [("a", 20), ("b", 2)], [("a", 1), ("b", 13), ("c", 9)], [("a", 7), ("b", 1)],
        [("b", 1), ("d", 2), ("a", 1)], [("d", 30), ("a", 1), ("b", 1)], [("a", 31)],
        [("b", 15), ("d", 1)], [("d", 14), ("e", 2)], [("f", 1)],
    ]
    steps = []
    for i, group in enumerate(plan):
        entries = [entry(k, n) for k, n in group]
        ended = [k for k, _ in group if at[k] == len(seqs[k])]
        steps.append({"step": i, "entries": entries, "end": ended})
    assert all(at[k] == len(v) for k, v in seqs.items())
    compare(collect(s, steps), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
def test_long_decoding_through_graphs(models, dtype):
    """Three hundred single tokens after a short prompt, two requests side by side (the steps of
    single tokens are captured into a graph and replayed, the routing of the experts with
    them), one of them starting later; the chunks of 48 positions pass many times."""
    folder, cfg, weights, page = models["B"]
    V = cfg["vocab"]
    seqs = {"a": random_tokens(330, V, 7), "b": random_tokens(290, V, 8)}
    want = {k: oracle("B", cfg, weights, v) for k, v in seqs.items()}
    s = session_for(folder, dtype, page, 704)
    assert s.model.graph_safe()
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": seqs["a"][:30], "want": [29]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": seqs["a"][30:31], "want": [0]},
                                     {"id": "b", "tokens": seqs["b"][:10], "want": [9]}], "end": []}]
    for i in range(280):
        steps.append({"step": 2 + i, "entries": [{"id": "a", "tokens": seqs["a"][31 + i: 32 + i], "want": [0]},
                                                 {"id": "b", "tokens": seqs["b"][10 + i: 11 + i], "want": [0]}],
                      "end": []})
    got = collect(s, steps)
    assert s.runner.graph_replays > 200
    compare(got, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
def test_the_stream_after_every_layer_run(models, dtype):
    """The float32 stream itself, layer run by layer run, against the plain model's: a step of one
    whole prompt with a hook on the blocks."""
    folder, cfg, weights, page = models["A"]
    tokens = random_tokens(40, cfg["vocab"], 21)
    _, layers = plain.vovalix_forward(cfg, weights, tokens, return_layers=True)
    s = session_for(folder, dtype, page, 64)
    seen = []
    for block in s.model.blocks:
        inner = block.forward

        def hooked(delta, residual, ctx, call, next_block=None, inner=inner):
            out = inner(delta, residual, ctx, call, next_block=next_block)
            assert out is None  # nothing stays pending: the stream is complete after the layer
            seen.append(residual[: ctx.num_tokens].detach().double().cpu().clone())
            return out

        block.forward = hooked
    s.run_step({"step": 0, "entries": [{"id": "a", "tokens": tokens, "want": [39]}], "end": ["a"]})
    assert len(seen) == len(cfg["layers"])
    limit = 1e-4 if dtype == torch.float32 else 5e-2
    for i, got in enumerate(seen):
        err = float((got - layers[i]).pow(2).mean().sqrt() / layers[i].pow(2).mean().sqrt())
        assert err < limit, f"layer run {i}: {err:.3e}"


@pytest.mark.parametrize("seed", [0, 6, 9, 21, 23, 27, 34, 56])
def test_configurations_drawn_at_random(tmp_path, seed):
    """Models whose every size, constant and layer order is drawn from a seed (widths that 8 does not
    divide, values wider than keys, chunks of 7 to 128 positions, one to twelve experts, borrowed
    layers, layers without a feed-forward), in float32, where the engine and the plain model agree
    to rounding whatever the routers choose: two requests side by side, portions, then single tokens."""
    import random

    from tests.vovalix_helpers import random_config

    cfg = random_config(random.Random(seed))
    folder = make_model_dir(tmp_path / "drawn", cfg, seed=seed)
    c, w = plain.load_model_folder(folder)
    seqs = {"a": random_tokens(150, cfg["vocab"], seed + 1), "b": random_tokens(70, cfg["vocab"], seed + 2)}
    want = {k: plain.vovalix_forward(c, w, v) for k, v in seqs.items()}
    s = session_for(folder, torch.float32, 16, 320, max_num_seqs=4)
    at = {"a": 0, "b": 0}
    steps = []
    for who, count in [("a", 37), ("b", 2), ("a", 50), ("b", 33)] + [("ab", 1)] * 30 + [("a", 33), ("b", 5)]:
        entries = []
        for k in who:
            lo, hi = at[k], min(at[k] + count, len(seqs[k]))
            if hi > lo:
                entries.append({"id": k, "tokens": seqs[k][lo:hi], "want": list(range(hi - lo))})
                at[k] = hi
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": [k for k in who if at[k] == len(seqs[k])]})
    got = collect(s, steps)
    assert len(got) == 220
    compare(got, want, torch.float32)


def test_attention_with_a_bias_and_chunks_runs_where_it_is_meant_to(models):
    """In bfloat16 with keys and values of 64 the chunked, biased attention takes the matrix-core
    kernels (portions and single tokens); in float32 the general kernel."""
    from kvcore_amd.ops import library as ops

    folder, cfg, weights, page = models["B"]
    m = cfg["layers"][1]["mixer"]
    assert ops.prefill_attention_supported(m["heads"], m["kv_heads"], m["dim"], page, torch.bfloat16)
    assert ops.decode_attention_supported(m["heads"], m["kv_heads"], m["dim"], page, torch.bfloat16)
    s = session_for(folder, torch.bfloat16, page, 128)
    tokens = random_tokens(71, cfg["vocab"], 9)
    s.run_step({"step": 0, "entries": [{"id": "a", "tokens": tokens[:70], "want": [69]}], "end": []})
    assert ops.last_variant("prefill_attention").startswith("prefill_attention_kernel")
    s.run_step({"step": 1, "entries": [{"id": "a", "tokens": tokens[70:], "want": [0]}], "end": ["a"]})
    assert ops.last_variant("decode_attention").startswith("decode_attention")


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_greedy_generation_through_the_engine(models, name, dtype):
    """``LLMEngine.generate`` with the scheduler cutting prompts into portions of 16 tokens:
    every generated token is the plain model's greedy choice given the tokens before it (a
    choice is skipped where the plain model's two best logits lie closer than rounding
    can tell apart)."""
    from kvcore_amd import CacheConfig, KVCoreConfig, ModelConfig, SamplingParams, SchedulerConfig
    from kvcore_amd.engine.llm_engine import GenerationRequest, LLMEngine

    folder, cfg, weights, page = models[name]
    V = cfg["vocab"]
    config = KVCoreConfig(
        model_config=ModelConfig(model=str(folder), dtype="float32" if dtype == torch.float32 else "bfloat16",
                                 max_model_len=128),
        cache_config=CacheConfig(block_size=page, num_gpu_blocks=40 if page >= 8 else 80),
        scheduler_config=SchedulerConfig(max_num_seqs=3, max_num_scheduled_tokens=24,
                                         long_prefill_token_threshold=16))
    engine = LLMEngine(config)
    prompts = {"r0": random_tokens(37, V, 11), "r1": random_tokens(5, V, 12), "r2": random_tokens(50, V, 13),
               "r3": random_tokens(18, V, 14), "r4": random_tokens(1, V, 15)}
    params = SamplingParams(max_tokens=12, temperature=0.0)
    outs = engine.generate([GenerationRequest(k, params, prompt_token_ids=tuple(v)) for k, v in prompts.items()])
    by_id = {o.request_id: list(o.output_token_ids) for o in outs}
    assert set(by_id) == set(prompts)
    margin = 1e-4 if dtype == torch.float32 else 5e-2
    checked = 0
    for rid, prompt in prompts.items():
        gen = by_id[rid]
        assert len(gen) == 12
        logits = plain.vovalix_forward(cfg, weights, prompt + gen)
        for i, tok in enumerate(gen):
            row = logits[len(prompt) + i - 1]
            top = torch.topk(row, 2).values
            if float(top[0] - top[1]) < margin * float(row.std()):
                continue
            assert int(torch.argmax(row)) == tok, f"{rid}: token {i}"
            checked += 1
    assert checked > 40


def test_command_lines(models, tmp_path):
    """``bin/kvcore_offline_batch`` generates with a Vovalix folder, and ``bin/trace_run``
    replays steps on it (on a folder whose config.json leaves the decay's rank to the tensors'
    shapes) and writes logits that match the plain model's."""
    import json
    import shutil
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    repo = Path(__file__).resolve().parent.parent
    folder, cfg, weights, page = models["A"]
    cmd = [sys.executable, str(repo / "bin" / "kvcore_offline_batch"), "--model", str(folder),
           "--dtype", "float32", "--prompt-lens", "7,16", "--max-tokens", "5", "--seed", "3",
           "--max-num-seqs", "4", "--max-num-scheduled-tokens", "32", "--num-gpu-blocks", "32",
           "--block-size", str(page), "--max-model-len", "128",
           "--ignore-eos", "--log-level", "WARNING", "--no-log-file"]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=240)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.count("finish_reason=length") == 2

    bare = tmp_path / "bare"
    shutil.copytree(folder, bare)
    stripped = json.loads((bare / "config.json").read_text())
    for layer in stripped["layers"]:
        layer["mixer"].pop("rank", None)
    (bare / "config.json").write_text(json.dumps(stripped))
    tokens = random_tokens(21, cfg["vocab"], 17)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": tokens[:13], "want": [0, 12]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": tokens[13:15], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": tokens[15:], "want": [5]}], "end": ["x"]}]
    out_dir = tmp_path / "logits"
    cmd = [str(repo / "bin" / "trace_run"), "--model", str(bare), "--dtype", "float32", "--out", str(out_dir),
           "--max-tokens", "64", "--block-size", str(page)]
    proc = subprocess.run(cmd, input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True,
                          text=True, timeout=240)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    assert not (out_dir / "1.f32").exists()
    want = oracle("A", cfg, weights, tokens)
    got = {("x", 0): torch.from_numpy(np.fromfile(out_dir / "0.f32", dtype="<f4").reshape(2, -1)[0]).double(),
           ("x", 12): torch.from_numpy(np.fromfile(out_dir / "0.f32", dtype="<f4").reshape(2, -1)[1]).double(),
           ("x", 20): torch.from_numpy(np.fromfile(out_dir / "2.f32", dtype="<f4").reshape(1, -1)[0]).double()}
    compare(got, {"x": want}, torch.float32)
