"""The Taluvik decoder in the engine against the plain implementation of tests/plain/taluvik.py:
every mechanism alone, whole prompts against decoding token by token, portions down to two tokens,
mixed batches with pages and state slots that are used again, long decoding from recorded graphs,
and greedy generation through ``LLM.generate`` and the scheduler; on three small configurations that
differ in every size, in 32-bit and in bfloat16."""

import math

import pytest
import torch

from . import schedules
from . import taluvik_models as models
from .helpers import random_tokens
from .plain import taluvik as plain
from .test_gpu_engine import run_trace

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [70, 41, 100, 35, 50, 33], "B": [66, 40, 130, 35, 90], "C": [45, 150, 37, 64, 120]}
#: distances are measured as a replay of a trace is judged: the difference of two rows of logits with
#: its mean taken off, root mean square over the vocabulary, over the root mean square of the truth
FP32_TOL = 2e-5
BF16_TOL = 4e-2


def distance(got: torch.Tensor, truth: torch.Tensor, scale: float) -> float:
    d = got.double() - truth.double()
    d = d - d.mean()
    return float(d.pow(2).mean().sqrt()) / scale


def truth_of(cfg, weights, requests):
    w64 = {k: v.double() for k, v in weights.items()}
    out = {rid: plain.forward(cfg, w64, toks) for rid, toks in requests.items()}
    scale = float(torch.cat([(t - t.mean(-1, keepdim=True)).flatten() for t in out.values()]).pow(2).mean().sqrt())
    return out, scale


class Case:
    def __init__(self, name, tmp):
        from torchllms_amd.engine import Engine

        self.name = name
        self.folder = models.make_folder(tmp / name, models.CONFIGS[name], seed=11)
        self.cfg, self.weights = models.read_folder(self.folder)
        self.requests = {f"r{i}": random_tokens(n, self.cfg["vocab"], 100 + i) for i, n in enumerate(LENGTHS[name])}
        self.truth, self.scale = truth_of(self.cfg, self.weights, self.requests)
        self.traces = {
            "whole": schedules.whole(self.requests),
            "tail": schedules.tail(self.requests),
            "portions": schedules.portions(self.requests),
            "mixed": schedules.mixed(self.requests),
        }
        page = models.PAGE_SIZE[name]
        pool_tokens = max(schedules.max_live_tokens(t) for t in self.traces.values())
        self.engines = {
            dt: Engine.from_folder(self.folder, dtype=dt, page_size=page, num_pages=-(-pool_tokens // page), max_seqs=4)
            for dt in ("float32", "bfloat16")
        }
        self._results = {}

    def result(self, dtype, schedule):
        key = (dtype, schedule)
        if key not in self._results:
            self._results[key] = run_trace(self.engines[dtype], self.traces[schedule])
        return self._results[key]

    def worst(self, result):
        worst, where = 0.0, None
        for (rid, pos), row in result.items():
            e = distance(row, self.truth[rid][pos], self.scale)
            if not e <= worst:
                worst, where = e, (rid, pos)
        return worst, where


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("taluvik")
    return {name: Case(name, tmp) for name in models.CONFIGS}


@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_float32_matches_the_plain_model(cases, name, schedule):
    case = cases[name]
    got = case.result("float32", schedule)
    assert len(got) == sum(len(t) for t in case.requests.values())
    err, where = case.worst(got)
    assert err < FP32_TOL, f"{name}/{schedule}: first look at {where}, distance {err}"


@pytest.mark.parametrize("schedule", ["tail", "portions", "mixed"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_float32_does_not_depend_on_the_schedule(cases, name, schedule):
    """Every 32-bit kernel adds in an order fixed by the element it computes (the recurrences token by
    token, the attention block by block of 64 keys), so cutting, batching, pages and slots change no bit."""
    case = cases[name]
    ref = case.result("float32", "whole")
    got = case.result("float32", schedule)
    diff = sorted(k for k in ref if not torch.equal(ref[k], got[k]))
    assert not diff, f"{name}/{schedule}: {len(diff)} positions differ, first {diff[0]}"


@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_bfloat16_stays_within_rounding(cases, name, schedule):
    case = cases[name]
    got = case.result("bfloat16", schedule)
    err, where = case.worst(got)
    assert err < BF16_TOL, f"{name}/{schedule}: first look at {where}, distance {err}"
    mean = sum(distance(row, case.truth[rid][pos], case.scale) for (rid, pos), row in got.items()) / len(got)
    assert mean < BF16_TOL / 3, f"{name}/{schedule}: mean distance {mean}"


# ----------------------------------------------------------------------------- every mechanism alone
ALONE = {
    "attention": models.layer("attention", models.attention(4, 2, 32, 48, 20, 16, 0.25, 6.0)),
    "attention_whole_head_rotated": models.layer("attention", models.attention(3, 3, 16, 16, 16, 9, 0.5, 30.0,
                                                 scaling={"factor": 4.0, "low": 1.0, "high": 4.0, "original": 16})),
    # keys and values of one head size that the matrix-core attention kernels take (bfloat16 runs those), with a
    # cap low enough to bend most scores
    "attention_matrix_cores_64": models.layer("attention", models.attention(8, 2, 64, 64, 32, 48, 0.6, 4.0)),
    "attention_matrix_cores_128": models.layer("attention", models.attention(4, 1, 128, 128, 64, 100, 0.4, 5.0, base=300.0)),
    "attention_matrix_cores_256": models.layer("attention", models.attention(2, 1, 256, 256, 128, 70, 0.05, 12.0)),
    "attention_matrix_cores_32": models.layer("attention", models.attention(16, 1, 32, 32, 32, 64, 0.7, 8.0)),
    "delta": models.layer("delta", {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 40, "conv": 4}),
    "delta_wide": models.layer("delta", {"heads": 1, "kv_heads": 1, "dim": 256, "vdim": 64, "conv": 2}),
    "delta_odd": models.layer("delta", {"heads": 3, "kv_heads": 1, "dim": 18, "vdim": 70, "conv": 3}),
    "mamba1": models.layer("mamba1", {"inner": 72, "state": 24, "dt_rank": 6, "conv": 3}),
    "mamba1_many_states": models.layer("mamba1", {"inner": 40, "state": 100, "dt_rank": 8, "conv": 6}),
    # a step-size rank that the decode products for 17 to 128 rows take (K a multiple of 128), read as a view of columns
    "mamba1_wide_rank": models.layer("mamba1", {"inner": 64, "state": 16, "dt_rank": 128, "conv": 4}),
    "feed_forward": models.layer("mamba1", {"inner": 8, "state": 1, "dt_rank": 1, "conv": 1}, ff=136),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("what", sorted(ALONE))
def test_a_mechanism_alone(tmp_path, what, dtype):
    """A model of one layer with that mixer and no feed-forward (or hardly a mixer and a feed-forward),
    a prompt in one step and, in a second request, the same tokens in portions and one by one."""
    from torchllms_amd.engine import Engine, StepEntry

    folder = models.make_folder(tmp_path / what, models.single_layer(ALONE[what]), seed=5)
    cfg, weights = models.read_folder(folder)
    tokens = random_tokens(275, cfg["vocab"], 9)
    truth, scale = truth_of(cfg, weights, {"r": tokens})
    page = 16 if what.endswith("_32") else 8  # (the matrix-core prefill kernel wants 512 / head size tokens a page)
    engine = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=640 // page, max_seqs=2)
    engine.admit("whole")
    whole = engine.step([StepEntry("whole", tokens, list(range(len(tokens))))]).cpu()
    engine.admit("cut")
    rows, at = [], 0
    for n in (5, 2, 30, 1, 1, 1, 17, 2, 1, 1, 13, 1, 150, 1, 1, 47, 1):
        rows.append(engine.step([StepEntry("cut", tokens[at : at + n], list(range(n)))]).cpu())
        at += n
    assert at == len(tokens)
    cut = torch.cat(rows)
    tol = FP32_TOL if dtype == "float32" else BF16_TOL
    for name, got in (("whole", whole), ("cut", cut)):
        worst = max(distance(got[i], truth["r"][i], scale) for i in range(len(tokens)))
        assert worst < tol, f"{what}/{name}: distance {worst}"
    if dtype == "float32":
        assert torch.equal(whole, cut)


# ----------------------------------------------------------------------------- attention: edges made visible
def _paged(keys: torch.Tensor, page_size: int, order):
    """Keys [n, H, d] into pages [pages, H, page_size, d] handed out in ``order``; returns pages and block table."""
    n, H, d = keys.shape
    blocks = -(-n // page_size)
    pages = torch.zeros((len(order), H, page_size, d), dtype=keys.dtype, device=keys.device)
    for b in range(blocks):
        rows = keys[b * page_size : (b + 1) * page_size]
        pages[order[b], :, : rows.shape[0]] = rows.transpose(0, 1)
    return pages, torch.tensor([order[:blocks]], dtype=torch.int32, device=keys.device)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("form", ["alone", "tile", "split"])
def test_one_key_that_stands_out_at_every_edge(form, dtype):
    """The plain attention kernel with chunks, a cap, sinks and values narrower than keys, on inputs in
    which one key has a score far above all others.  Queries are placed so that this key is the first of
    their chunk, the last of the chunk before, at a page's border, far back, or the query itself: the
    output is that key's value (less the sink's share) or hardly any of it.  All three launches of the kernel."""
    from torchllms_amd.kernels import ops

    dev = "cuda:0"
    H, G, d, dv, chunk, page = 4, 2, 32, 16, 48, 16
    n = 300
    g = torch.Generator().manual_seed(3)
    k = torch.randn((n, G, d), generator=g) * 0.3
    v = torch.randn((n, G, dv), generator=g)
    special = [0, 47, 48, 95, 96, 143, 144, 160, 239, 240, 287]  # chunk and page borders among them
    direction = torch.randn(d, generator=g)
    direction = direction / direction.norm()
    for j in special:
        k[j] += 6.0 * direction * (1 + 0.01 * j)
    sinks = torch.tensor([0.5, -1.0, 2.0, 0.0])
    scale, cap = 1.3, 9.0
    if form == "alone":
        query_at = [0, 1, 46, 47, 48, 49, 94, 95, 96, 97, 143, 144, 159, 160, 161, 239, 240, 241, 286, 287, 288, 299]
    elif form == "tile":
        query_at = list(range(n))
    else:
        query_at = [299, 287, 241, 240]  # few tokens, each a request of its own length: the split form
    q = torch.randn((len(query_at), H, d), generator=g) * 0.2 + 4.0 * direction
    # truth in 64-bit from the formula
    want = torch.zeros((len(query_at), H, dv), dtype=torch.float64)
    kd, vd, qd = k.to(dtype).double(), v.to(dtype).double(), q.to(dtype).double()
    for r, p in enumerate(query_at):
        lo = p - p % chunk
        for h in range(H):
            s = (kd[lo : p + 1, h // 2] @ qd[r, h]) * scale
            s = cap * torch.tanh(s / cap)
            m = max(float(s.max()), float(sinks[h]))
            e = torch.exp(s - m)
            want[r, h] = (e / (e.sum() + math.exp(float(sinks[h]) - m))) @ vd[lo : p + 1, h // 2]
    order = torch.randperm(32, generator=g).tolist()
    k_pages, bt = _paged(k.to(dtype).to(dev), page, order)
    v_pages, _ = _paged(v.to(dtype).to(dev), page, order)
    qkv = q.to(dtype).reshape(len(query_at), H * d).to(dev).contiguous()
    seq = torch.zeros(len(query_at), dtype=torch.int32, device=dev)
    pos = torch.tensor(query_at, dtype=torch.int32, device=dev)
    kw = dict(softcap=cap, chunk=chunk, sinks=sinks.to(dev), v_head_dim=dv)
    if form == "split":
        got = ops.attention_generic_split(qkv, H, G, d, k_pages, v_pages, seq, pos, bt, 0, scale, longest=chunk, **kw)
    else:
        got = ops.attention_generic(qkv, H, G, d, k_pages, v_pages, seq, pos, bt, 0, scale, **kw)
    got = got.float().cpu().double().reshape(len(query_at), H, dv)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert (got - want).abs().max() < tol, f"first wrong query at position {query_at[int((got - want).abs().amax((1, 2)).argmax())]}"
    # the inputs do what they are made for: the query right behind a chunk's first key gives nearly all
    # of its weight to that key, and the query on the chunk's first position cannot see the key before it
    if 49 in query_at:
        near = want[query_at.index(49), 1]
        assert (near - vd[48, 0] * (near @ vd[48, 0]) / (vd[48, 0] @ vd[48, 0])).norm() < 0.2 * near.norm()
    # the three launches agree bit for bit
    if form == "tile":
        few = [0, 47, 48, 49, 143, 144, 299]
        rows = torch.tensor(few, device=dev)
        alone = ops.attention_generic(qkv[rows].contiguous(), H, G, d, k_pages, v_pages, seq[: len(few)].contiguous(),
                                      pos[rows].contiguous(), bt, 0, scale, **kw)
        split = ops.attention_generic_split(qkv[rows].contiguous(), H, G, d, k_pages, v_pages, seq[: len(few)].contiguous(),
                                            pos[rows].contiguous(), bt, 0, scale, longest=chunk, **kw)
        tile = ops.attention_generic(qkv, H, G, d, k_pages, v_pages, seq, pos, bt, 0, scale, **kw)[rows]
        assert torch.equal(alone, tile) and torch.equal(alone, split)


# ----------------------------------------------------------------------------- state that is carried, freed and used again
def test_slots_and_pages_that_are_used_again_start_clean(tmp_path):
    """Two slots, few pages: six requests pass through them one after the other and side by side, each
    beside a neighbour that is at another place of its own sequence; every one must come out as alone."""
    from torchllms_amd.engine import Engine

    folder = models.make_folder(tmp_path / "m", models.CONFIGS["A"], seed=2)
    cfg, weights = models.read_folder(folder)
    requests = {f"q{i}": random_tokens(n, cfg["vocab"], 50 + i) for i, n in enumerate([30, 55, 18, 41, 26, 60])}
    truth, scale = truth_of(cfg, weights, requests)
    steps = schedules.mixed(requests, max_live=2)
    pool = schedules.max_live_tokens(steps, round_to=8)
    engine = Engine.from_folder(folder, dtype="float32", page_size=8, num_pages=pool // 8, max_seqs=2)
    got = run_trace(engine, steps)
    worst = max(distance(row, truth[rid][pos], scale) for (rid, pos), row in got.items())
    assert worst < FP32_TOL, worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_from_recorded_steps(tmp_path, dtype):
    """A short prompt and 400 tokens one by one, two requests side by side: the decode steps are
    recorded as graphs after a few, and replayed; states and histories move on with every replay,
    chunks begin and end, and the windows of the convolutions hold tokens of the steps before."""
    from torchllms_amd.engine import Engine, StepEntry

    folder = models.make_folder(tmp_path / "m", models.CONFIGS["B"], seed=8)
    cfg, weights = models.read_folder(folder)
    requests = {"a": random_tokens(410, cfg["vocab"], 1), "b": random_tokens(425, cfg["vocab"], 2)}
    truth, scale = truth_of(cfg, weights, requests)
    engine = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=64, max_seqs=2)
    assert engine.graphs is not None
    heads = {"a": 10, "b": 25}
    for rid, toks in requests.items():
        engine.admit(rid)
        engine.step([StepEntry(rid, toks[: heads[rid]], [])])
    tol = FP32_TOL if dtype == "float32" else BF16_TOL
    worst = 0.0
    for i in range(400):
        entries = [StepEntry(rid, [requests[rid][heads[rid] + i]], [0]) for rid in ("a", "b")]
        logits = engine.step(entries).cpu()
        for row, rid in zip(logits, ("a", "b")):
            worst = max(worst, distance(row, truth[rid][heads[rid] + i], scale))
    assert any(g.replays > 100 for g in engine.graphs.graphs.values())
    assert worst < tol, worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_beside_short_ones(tmp_path, dtype):
    """Prompts of several hundred tokens in one step, beside a short portion and a single token of
    other requests: in bfloat16 the selective scan cuts long rows into segments that run side by side
    (the last one shorter), and the delta rule's tiles and the attention's chunks end inside them."""
    from torchllms_amd.engine import Engine, StepEntry

    folder = models.make_folder(tmp_path / "m", models.CONFIGS["A"], seed=12)
    cfg, weights = models.read_folder(folder)
    requests = {"long": random_tokens(700, cfg["vocab"], 1), "mid": random_tokens(333, cfg["vocab"], 2),
                "short": random_tokens(40, cfg["vocab"], 3), "one": random_tokens(9, cfg["vocab"], 4)}
    truth, scale = truth_of(cfg, weights, requests)
    engine = Engine.from_folder(folder, dtype=dtype, page_size=8, num_pages=160, max_seqs=4)
    for rid in requests:
        engine.admit(rid)
    engine.step([StepEntry("short", requests["short"][:31], []), StepEntry("one", requests["one"][:8], [])])
    wanted = {"long": [0, 63, 64, 255, 256, 639, 640, 699], "mid": [0, 100, 320, 332], "short": list(range(9)), "one": [0]}
    entries = [StepEntry("long", requests["long"], wanted["long"]), StepEntry("one", requests["one"][8:], [0]),
               StepEntry("mid", requests["mid"], wanted["mid"]), StepEntry("short", requests["short"][31:], wanted["short"])]
    logits = engine.step(entries).cpu()
    tol = FP32_TOL if dtype == "float32" else BF16_TOL
    at = 0
    for e, base in zip(entries, (0, 8, 0, 31)):
        for w in e.want:
            d = distance(logits[at], truth[e.rid][base + w], scale)
            assert d < tol, f"{e.rid} at {base + w}: distance {d}"
            at += 1
    # and the states that the long rows left behind carry on
    more = engine.step([StepEntry("long", [5], [0]), StepEntry("mid", [7], [0])]).cpu()
    w64 = {k: v.double() for k, v in weights.items()}
    for row, (rid, tok) in zip(more, (("long", 5), ("mid", 7))):
        assert distance(row, plain.forward(cfg, w64, requests[rid] + [tok])[-1], scale) < tol


def test_greedy_generation_through_the_entry_point(tmp_path):
    """``LLM.generate``: the scheduler admits, cuts prompts into portions under a small token budget,
    decodes everybody together and frees; the tokens are the plain model's."""
    from torchllms_amd.inference import LLM

    folder = models.make_folder(tmp_path / "m", models.CONFIGS["A"], seed=4)
    cfg, weights = models.read_folder(folder)
    w64 = {k: v.double() for k, v in weights.items()}
    prompts = [random_tokens(n, cfg["vocab"], 40 + n) for n in (5, 37, 1, 64, 22)]
    new = 20

    def plain_greedy(prompt):
        toks = list(prompt)
        for _ in range(new):
            toks.append(int(plain.forward(cfg, w64, toks)[-1].argmax()))
        return toks[len(prompt):]

    llm = LLM(str(folder), precision="float32", max_len=128, max_bsz=3, page_size=8, max_num_batched_tokens=24)
    results = llm.generate(prompt_token_ids=prompts, temperature=0.0, max_new_tokens=new)
    for p, r in zip(prompts, results):
        assert r.token_ids == plain_greedy(p)
    llm.engine.cache.check_invariants()
    assert llm.engine.cache.live == []
    # in bfloat16 the first token of each request is the one the plain model rates highest or next to it
    llm16 = LLM(str(folder), precision="bfloat16", max_len=128, max_bsz=3, page_size=8)
    for p, r in zip(prompts, llm16.generate(prompt_token_ids=prompts, temperature=0.0, max_new_tokens=4)):
        logits = plain.forward(cfg, w64, p)[-1]
        assert logits[r.token_ids[0]] >= logits.max() - 0.05 * float(logits.std())


def test_a_preempted_request_starts_again_from_clean_state(tmp_path):
    """Too few pages for four requests: the scheduler takes the youngest off, gives its pages and its slot away and
    later computes it again from its prompt and what it had generated.  Its convolution histories and recurrent
    states must then start from zero again: the sampled tokens are those of the run with room for everybody."""
    from torchllms_amd.inference import LLM

    folder = models.make_folder(tmp_path / "m", models.CONFIGS["A"], seed=9)
    cfg, _ = models.read_folder(folder)
    prompts = [random_tokens(n, cfg["vocab"], 80 + n) for n in (30, 25, 28, 21)]
    ample = LLM(str(folder), precision="float32", max_len=96, max_bsz=4, page_size=8)
    want = ample.generate(prompt_token_ids=prompts, temperature=0.8, max_new_tokens=30, seed=7)
    tight = LLM(str(folder), precision="float32", max_len=96, max_bsz=4, page_size=8, num_pages=20)  # 160 places for 224 tokens
    got = tight.generate(prompt_token_ids=prompts, temperature=0.8, max_new_tokens=30, seed=7)
    assert tight.last_stats["preemptions"] > 0
    assert [r.token_ids for r in got] == [r.token_ids for r in want]
    tight.engine.cache.check_invariants()


def test_generate_command_line_with_random_weights(tmp_path):
    """The generate program given nothing but a config.json: ``--random-weights --seed`` draws the weights that
    ``write_model_folder`` would write for that seed, so the plain model can say which tokens to expect."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    from torchllms_amd.config import TaluvikConfig
    from torchllms_amd.weights import write_model_folder

    root = Path(__file__).resolve().parent.parent
    folder = tmp_path / "only_config"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(models.CONFIGS["B"]))
    prompt = random_tokens(13, models.CONFIGS["B"]["vocab"], 21)
    proc = subprocess.run(
        [sys.executable, "-m", "torchllms_amd.inference.generate", "--model", str(folder), "--dtype", "float32", "--random-weights",
         "--seed", "7", "--max-new-tokens", "6", "--prompt-ids", *map(str, prompt)],
        capture_output=True, text=True, cwd=root, timeout=300,
    )
    assert proc.returncode == 0, proc.stderr[-2000:]
    got = [int(t) for t in proc.stdout.split()[-6:]]
    written = write_model_folder(tmp_path / "written", TaluvikConfig.from_dict(models.CONFIGS["B"]), seed=7, dtype=torch.float32)
    cfg, weights = models.read_folder(written)
    w64 = {k: v.double() for k, v in weights.items()}
    toks = list(prompt)
    for _ in range(6):
        toks.append(int(plain.forward(cfg, w64, toks)[-1].argmax()))
    assert got == toks[len(prompt):]


def test_trace_replay_program(tmp_path):
    """``bin/trace_run`` as a process: steps in, logits files out, the plain model's values."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    root = Path(__file__).resolve().parent.parent
    folder = models.make_folder(tmp_path / "m", models.CONFIGS["C"], seed=6)
    cfg, weights = models.read_folder(folder)
    requests = {"x": random_tokens(50, cfg["vocab"], 1), "y": random_tokens(90, cfg["vocab"], 2), "z": random_tokens(20, cfg["vocab"], 3)}
    truth, scale = truth_of(cfg, weights, requests)
    steps = schedules.mixed(requests, max_live=2)
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, str(root / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32", "--out", str(out),
         "--max-tokens", str(schedules.max_live_tokens(steps))],
        input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600,
    )
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done ")] == [f"done {i}" for i in range(len(steps))]
    for step, rows in zip(steps, schedules.positions_of(steps)):
        got = torch.from_numpy(np.fromfile(out / f"{step['step']}.f32", dtype="<f4").reshape(len(rows), -1))
        for row, (rid, pos) in zip(got, rows):
            assert distance(row, truth[rid][pos], scale) < FP32_TOL


# ----------------------------------------------------------------------------- random configurations
def random_config(seed: int) -> dict:
    """A Taluvik configuration drawn from a seed: every size, constant and the order of layers."""
    import random

    rng = random.Random(seed)
    width = rng.choice([40, 64, 72, 96, 128, 160])
    layers = []
    for _ in range(rng.randint(2, 5)):
        kind = rng.choice(["attention", "delta", "mamba1"])
        ff = rng.choice([None, 48, 100, 136])
        if layers and rng.random() < 0.25:
            owner = rng.choice([i for i, l in enumerate(layers) if "weights_of" not in l])
            layers.append(dict(layers[owner], weights_of=owner))
            continue
        if kind == "attention":
            kv = rng.choice([1, 2, 3])
            heads = kv * rng.choice([1, 2, 4])
            dim = rng.choice([16, 24, 32, 64, 128])
            vdim = rng.choice([dim, dim, 16, 40, 64])
            rot = rng.choice([0, dim // 2, dim]) // 2 * 2
            scaling = rng.choice([None, {"factor": rng.choice([2.0, 8.0]), "low": 1.0, "high": rng.choice([2.0, 4.0]), "original": rng.choice([16, 64])}])
            mixer = models.attention(heads, kv, dim, vdim, rot, rng.choice([5, 16, 33, 64, 100]), rng.choice([0.1, 0.3, 1.0]) * 32 / dim,
                                     rng.choice([2.0, 10.0, 50.0]), base=rng.choice([100.0, 10000.0, 500000.0]), scaling=scaling)
        elif kind == "delta":
            kv = rng.choice([1, 2, 3])
            mixer = {"heads": kv * rng.choice([1, 2]), "kv_heads": kv, "dim": rng.choice([8, 20, 32, 64, 128, 192]),
                     "vdim": rng.choice([8, 24, 32, 64, 100]), "conv": rng.choice([1, 2, 3, 4, 5])}
        else:
            mixer = {"inner": rng.choice([24, 64, 100, 256]), "state": rng.choice([1, 4, 8, 16, 24, 48, 64, 130]),
                     "dt_rank": rng.choice([1, 3, 8, 16, 40]), "conv": rng.choice([1, 2, 3, 4, 7])}
        layers.append(models.layer(kind, mixer, ff=ff))
    return {"architecture": "Taluvik", "vocab": rng.choice([50, 97, 256, 301]), "width": width,
            "embedding": {"scale": rng.choice([1.0, 0.5, 12.0])}, "norm": {"eps": rng.choice([1e-5, 1e-6, 1e-3])},
            "residual_mult": rng.choice([1.0, 0.3, 0.8]), "layers": layers}


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(tmp_path, seed):
    """Sizes nobody chose: a prompt whole, and the same tokens in portions, single tokens and beside a second
    request, in both dtypes, against the plain model."""
    import random

    from torchllms_amd.engine import Engine, StepEntry

    cfg_dict = random_config(1000 + seed)
    folder = models.make_folder(tmp_path / "m", cfg_dict, seed=seed)
    cfg, weights = models.read_folder(folder)
    rng = random.Random(seed)
    requests = {"a": random_tokens(rng.randint(120, 330), cfg["vocab"], seed), "b": random_tokens(rng.randint(20, 90), cfg["vocab"], seed + 50)}
    truth, scale = truth_of(cfg, weights, requests)
    page = rng.choice([4, 8, 16, 32])
    # (bfloat16: what rounding alone does depends on the model that was drawn.  Mean distances are 0.003 to 0.006 for
    # most seeds and up to 0.03 for a few: attention with scores of +-30 turns the 0.4% that bfloat16 leaves of a
    # query into tens of percent of a weight, five layers on a stream as small as a layer's own addition pass an
    # error on enlarged, and the first tokens of a delta layer read out a small difference divided by its own size.
    # Traced layer by layer for two such seeds: every layer adds 0.3 to 1.5% of its own output, none more.  So the
    # 32-bit comparison above is the sharp one here; bfloat16 is held to what a fault of its own kernels would
    # exceed: a position five times the hand-made configurations' bound, one in fifty positions twice, the mean once.)
    for dtype, tol in (("float32", FP32_TOL), ("bfloat16", 5 * BF16_TOL)):
        seen = []
        engine = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=2 * (-(-420 // page)) + 4, max_seqs=3)
        engine.admit("w")
        whole = engine.step([StepEntry("w", requests["a"], list(range(len(requests["a"]))))]).cpu()
        engine.free("w")
        for i, row in enumerate(whole):
            d = distance(row, truth["a"][i], scale)
            seen.append(d)
            assert d < tol, f"{dtype} whole at {i}: {d}  {cfg_dict}"
        at = {"a": 0, "b": 0}
        engine.admit("a")
        engine.admit("b")
        while at["a"] < len(requests["a"]) or at["b"] < len(requests["b"]):
            entries = []
            for rid in ("a", "b"):
                left = len(requests[rid]) - at[rid]
                if left and rng.random() < 0.8:
                    n = min(left, rng.choice([1, 1, 2, 3, 17, 40, 64, 130]))
                    entries.append(StepEntry(rid, requests[rid][at[rid] : at[rid] + n], list(range(n))))
            if not entries:
                continue
            logits = engine.step(entries).cpu()
            k = 0
            for e in entries:
                for w in e.want:
                    d = distance(logits[k], truth[e.rid][at[e.rid] + w], scale)
                    seen.append(d)
                    assert d < tol, f"{dtype} {e.rid} at {at[e.rid] + w} in a step of {[len(x.tokens) for x in entries]}: {d}  {cfg_dict}"
                    if dtype == "float32" and e.rid == "a":
                        assert torch.equal(logits[k], whole[at["a"] + w])
                    k += 1
                at[e.rid] += len(e.tokens)
        if dtype == "bfloat16":
            assert sum(seen) / len(seen) < BF16_TOL, f"mean distance {sum(seen) / len(seen)}  {cfg_dict}"
            assert sum(d > 2 * BF16_TOL for d in seen) <= len(seen) // 50, f"{sum(d > 2 * BF16_TOL for d in seen)} of {len(seen)} positions  {cfg_dict}"
        del engine


# ----------------------------------------------------------------------------- sizes of the order of a real model's layers
LARGER = {
    "architecture": "Taluvik", "vocab": 1000, "width": 1024, "embedding": {"scale": 4.0}, "norm": {"eps": 1e-5},
    "residual_mult": 0.5,
    "layers": [
        models.layer("mamba1", {"inner": 2048, "state": 16, "dt_rank": 64, "conv": 4}, ff=2816),
        models.layer("attention", models.attention(16, 4, 128, 128, 64, 256, 0.09, 30.0, base=500000.0,
                                                   scaling={"factor": 8.0, "low": 1.0, "high": 4.0, "original": 128}), ff=2816),
        models.layer("delta", {"heads": 8, "kv_heads": 4, "dim": 128, "vdim": 128, "conv": 4}, ff=2816),
        models.layer("attention", models.attention(16, 16, 64, 64, 64, 100, 0.125, 20.0), ff=2816),
    ],
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_of_larger_sizes(tmp_path, dtype):
    """Heads of 128 and 64 that the matrix-core attention kernels take, a delta rule of 128 by 128 (eight rows a lane,
    sixteen lanes a column, 16 and 32 columns a block), a scan over 2,048 channels in segments, products that the
    library, the streaming kernel and the kernel for 17 to 128 rows serve: a prompt of 700 tokens whole, then a
    second request in portions beside single tokens of the first, then sixteen requests decoding together."""
    from torchllms_amd.engine import Engine, StepEntry

    folder = models.make_folder(tmp_path / "m", LARGER, seed=21)
    cfg, weights = models.read_folder(folder)
    requests = {"a": random_tokens(740, cfg["vocab"], 1), "b": random_tokens(300, cfg["vocab"], 2)}
    requests.update({f"d{i}": random_tokens(40 + 3 * i, cfg["vocab"], 10 + i) for i in range(16)})
    truth, scale = truth_of(cfg, weights, requests)
    tol = FP32_TOL if dtype == "float32" else BF16_TOL
    engine = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=160, max_seqs=18)
    worst = 0.0

    def step(entries):
        nonlocal worst
        logits = engine.step(entries).cpu()
        k = 0
        for e in entries:
            base = engine.num_tokens(e.rid) - len(e.tokens)
            for w in e.want:
                worst = max(worst, distance(logits[k], truth[e.rid][base + w], scale))
                k += 1

    for rid in requests:
        engine.admit(rid)
    step([StepEntry("a", requests["a"][:700], list(range(0, 700, 7)) + [699])])
    at = 0
    for n in (130, 2, 64, 1, 33, 70):
        step([StepEntry("b", requests["b"][at : at + n], list(range(n))), StepEntry("a", [requests["a"][700 + at // 50]], [0])]
             if at < 250 and engine.num_tokens("a") == 700 + at // 50 else [StepEntry("b", requests["b"][at : at + n], list(range(n)))])
        at += n
    assert at == 300
    step([StepEntry(f"d{i}", requests[f"d{i}"][:-8], [len(requests[f"d{i}"]) - 9]) for i in range(16)])
    for j in range(8, 0, -1):
        step([StepEntry(f"d{i}", [requests[f"d{i}"][-j]], [0]) for i in range(16)])
    assert worst < tol, worst


@pytest.mark.parametrize("head_dim", [32, 64, 128, 256])
def test_matrix_core_attention_agrees_with_the_plain_kernel(head_dim):
    """The split-KV decode kernel and the tiled prefill kernel with a cap, chunks and sinks against the plain
    kernel on the same pages and queries: a prompt portion behind cached keys beside two single tokens, chunks
    that end inside the portion and inside a tile of keys."""
    from torchllms_amd.engine.context import upload
    from torchllms_amd.engine.layout import StepEntry, build_step_layout
    from torchllms_amd.kernels import ops
    from torchllms_amd.kernels.attention import paged_attention

    dev = "cuda:0"
    G = 2
    H = G * (4 if head_dim < 256 else 2)
    page, chunk = 16, 88
    entries = [StepEntry("p", [0] * 150, []), StepEntry("d", [0], []), StepEntry("e", [0], [])]
    starts = [70, 200, 87]
    tables = [[list(range(0, 14)), list(range(14, 27)), list(range(27, 33))]]
    layout = build_step_layout(entries, starts, [0, 1, 2], tables, [page])
    assert layout.n_decode == 2
    ctx = upload(layout, dev)
    g = torch.Generator().manual_seed(head_dim)
    qkv = torch.randn((152, H * head_dim), generator=g).to(torch.bfloat16).to(dev)
    k_pages = torch.randn((40, G, page, head_dim), generator=g).to(torch.bfloat16).to(dev)
    v_pages = torch.randn((40, G, page, head_dim), generator=g).to(torch.bfloat16).to(dev)
    extras = dict(softcap=6.0, chunk=chunk, sinks=torch.randn(H, generator=g).to(dev))
    scale = 2.5 / head_dim ** 0.5
    assert ops.decode_attention_supported(torch.bfloat16, H, G, head_dim)
    assert ops.prefill_attention_supported(torch.bfloat16, H, G, head_dim, page)
    fast = paged_attention(qkv, H, G, head_dim, k_pages, v_pages, ctx, 0, 0, scale, **extras).float()
    plain_out = ops.attention_generic(qkv, H, G, head_dim, k_pages, v_pages, ctx.token_seq, ctx.positions, ctx.block_tables[0],
                                      0, scale, v_head_dim=head_dim, **extras).float()
    assert (fast - plain_out).abs().max() < 0.03, (fast - plain_out).abs().max()
    # what the comparison would miss if both forgot the same thing: the plain kernel alone notices each of the three
    for change in (dict(extras, softcap=0.0), dict(extras, chunk=0), dict(extras, sinks=None)):
        other = ops.attention_generic(qkv, H, G, head_dim, k_pages, v_pages, ctx.token_seq, ctx.positions, ctx.block_tables[0],
                                      0, scale, v_head_dim=head_dim, **change).float()
        assert (other - plain_out).abs().max() > 0.1
