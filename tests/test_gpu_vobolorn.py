"""The Vobolorn decoder in the engine against the plain implementation of tests/plain/vobolorn.py: every
mechanism alone, whole prompts against decoding token by token, portions down to two tokens, mixed batches
with pages and slots that are used again, keys far back and at page borders, the steps of the query factor,
long decoding from recorded graphs, greedy generation through ``LLM.generate`` and the scheduler, and
configurations drawn from seeds; in 32-bit and in bfloat16."""

import math
import random

import pytest
import torch

from . import schedules
from . import vobolorn_models as models
from .helpers import random_tokens
from .plain import vobolorn as plain
from .test_gpu_engine import run_trace

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [70, 41, 100, 35, 50, 33], "B": [66, 40, 130, 35, 90], "C": [45, 150, 37, 64, 120]}
#: distances are measured as a replay of a trace is judged: the difference of two rows of logits with its mean
#: taken off, root mean square over the vocabulary, over the root mean square of the truth
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


def bfloat16_bounds(cfg, weights, requests, truth, scale):
    """``(worst, mean)`` distance that the engine may have from the truth in bfloat16: the plain model computed in
    bfloat16 throughout (its residual stream too, which the engine keeps in 32-bit) is the yardstick, so the engine has
    to be about as near as that or nearer; ``BF16_TOL`` where the plain model is nearer than that itself."""
    w16 = {k: v.bfloat16() for k, v in weights.items()}
    ds = []
    for rid, toks in requests.items():
        z = plain.forward(cfg, w16, toks)
        ds += [distance(z[i], truth[rid][i], scale) for i in range(len(toks))]
    return max(BF16_TOL, 1.25 * max(ds)), max(BF16_TOL / 3, 1.25 * sum(ds) / len(ds))


def float32_bound(cfg, weights, requests, truth, scale):
    """The distance that the engine may have from the truth in 32-bit: ``FP32_TOL``, or, where drawn weights make
    scores so sharp that the plain model computed in 32-bit is farther from the 64-bit truth than that itself,
    two and a half times the plain model's distance."""
    w32 = {k: v.float() for k, v in weights.items()}
    worst = 0.0
    for rid, toks in requests.items():
        z = plain.forward(cfg, w32, toks)
        worst = max(worst, max(distance(z[i], truth[rid][i], scale) for i in range(len(toks))))
    return max(FP32_TOL, 2.5 * worst)


class Case:
    def __init__(self, name, tmp):
        from torchllms_amd.engine import Engine

        self.name = name
        self.folder = models.make_folder(tmp / name, models.CONFIGS[name], seed=11)
        self.cfg, self.weights = models.read_folder(self.folder)
        self.requests = {f"r{i}": random_tokens(n, self.cfg["vocab"], 100 + i) for i, n in enumerate(LENGTHS[name])}
        self.truth, self.scale = truth_of(self.cfg, self.weights, self.requests)
        self.bf16_worst, self.bf16_mean = bfloat16_bounds(self.cfg, self.weights, self.requests, self.truth, self.scale)
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
    tmp = tmp_path_factory.mktemp("vobolorn")
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
    """Every 32-bit kernel adds in an order fixed by the element it computes (the attention block by block of
    64 keys, the products in groups of 16 along K, the per-head products of the latent layer with the same
    kernel head by head), so cutting, batching, pages and slots change no bit."""
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
    assert err < case.bf16_worst, f"{name}/{schedule}: first look at {where}, distance {err}"
    mean = sum(distance(row, case.truth[rid][pos], case.scale) for (rid, pos), row in got.items()) / len(got)
    assert mean < case.bf16_mean, f"{name}/{schedule}: mean distance {mean}"


# ----------------------------------------------------------------------------- every mechanism alone
ALONE = {
    "biases_and_gate": [models.layer(models.grouped("attention", 4, 2, 24, 40, 0.5))],
    "query_factor": [models.layer(models.grouped("attention_2", 3, 1, 20, 12, 0.6, q_temp=(0.7, 5)))],
    "query_factor_every_token": [models.layer(models.grouped("attention_2", 2, 2, 16, 16, 0.8, q_temp=(0.4, 1)))],
    "mixed_values": [models.layer(models.grouped("attention_2", 2, 1, 16, 24, 0.5, q_temp=(0.1, 9), v_mix=True)),
                     models.layer(models.grouped("attention", 6, 1, 8, 24, 0.9, v_mix=True)),
                     models.layer(models.grouped("attention_2", 1, 1, 32, 24, 0.4, q_temp=(0.1, 9), v_mix=True))],
    "latent": [models.layer(models.latent(3, 16, 8, 24, 12, 36, 0.4))],
    "latent_nothing_rotated": [models.layer(models.latent(2, 24, 0, 12, 20, 44, 0.3))],
    "latent_one_head_wide_rotation": [models.layer(models.latent(1, 8, 64, 8, 40, 16, 0.2, base=100.0))],
    "latent_wider_than_the_values_the_kernel_takes": [models.layer(models.latent(2, 16, 4, 16, 16, 260, 0.3))],
    # latent and rotated part together make rows that the matrix-core attention kernels take (bfloat16 runs those,
    # twelve heads in two calls at 256 channels)
    "latent_matrix_cores_256": [models.layer(models.latent(12, 16, 64, 16, 24, 192, 0.2))],
    "latent_matrix_cores_64": [models.layer(models.latent(5, 24, 16, 8, 20, 48, 0.3))],
    # heads of one size that the matrix-core attention kernels take (bfloat16 runs those)
    "matrix_cores_64": [models.layer(models.grouped("attention", 8, 2, 64, 64, 0.3, v_mix=True)),
                        models.layer(models.grouped("attention_2", 4, 2, 64, 64, 0.3, q_temp=(0.5, 20), v_mix=True))],
    "matrix_cores_128": [models.layer(models.grouped("attention_2", 4, 1, 128, 128, 0.2, q_temp=(0.3, 33)))],
    "matrix_cores_32": [models.layer(models.grouped("attention", 16, 1, 32, 32, 0.5))],
    "feed_forward": [models.layer(models.grouped("attention_2", 1, 1, 4, 4, 0.5, q_temp=(0.0, 1)), ff=136)],
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("what", sorted(ALONE))
def test_a_mechanism_alone(tmp_path, what, dtype):
    """A model of that mixer and no feed-forward (or hardly a mixer and a feed-forward), a prompt in one step
    and, in a second request, the same tokens in portions and one by one."""
    from torchllms_amd.engine import Engine, StepEntry

    cfg_dict = models.model(61, 64, 1e-5, ALONE[what], softcap=None if "latent" in what else 9.0)
    folder = models.make_folder(tmp_path / "m", cfg_dict, seed=5)
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
    tol = FP32_TOL if dtype == "float32" else bfloat16_bounds(cfg, weights, {"r": tokens}, truth, scale)[0]
    for name, got in (("whole", whole), ("cut", cut)):
        worst = max(distance(got[i], truth["r"][i], scale) for i in range(len(tokens)))
        assert worst < tol, f"{what}/{name}: distance {worst}"
    if dtype == "float32":
        assert torch.equal(whole, cut)


# ----------------------------------------------------------------------------- the kernels against torch in 32-bit
def _bf16_tol(dtype):
    return dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pairing", [0, 1])
def test_head_prepare_against_its_formulas(dtype, pairing):
    """A bias, the weighted norm over the first channels, rotation of a middle part, the query factor at the positions where
    it steps (just below, at and just above multiples of ``every``, and position 0), mixed values, pages."""
    from torchllms_amd.kernels import ops

    dev = "cuda:0"
    g = torch.Generator().manual_seed(1)
    H, G, dk, dv, extra = 5, 2, 44, 12, 7
    norm_dims, rot_off, rot = 30, 30, 14
    every, coef = 6, 0.37
    positions = [0, 1, 4, 5, 6, 10, 11, 12, 17, 599, 600, 5, 35, 36]
    n = len(positions)
    width = (H + G) * dk + G * dv + extra
    rows = torch.randn((n, width), generator=g).to(dtype)
    qw, kw = torch.rand(norm_dims, generator=g) + 0.5, torch.rand(norm_dims, generator=g) + 0.5
    v_first = torch.randn((n, G * dv), generator=g).to(dtype)
    lam = torch.tensor([0.3])
    inv_freq = 1.0 / (50.0 ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot))
    pos = torch.tensor(positions, dtype=torch.int32)
    ang = (pos.float()[:, None] * inv_freq[None, :]).double()  # (the angle is a 32-bit product, as in the engine)
    page_size, n_pages = 4, 9
    slots = torch.tensor([3, 0, 35, 9, 8, 17, 21, 22, 23, 1, 30, 31, 12, 2], dtype=torch.int32)

    heads_width = (H + G) * dk + G * dv
    bias = torch.randn(heads_width, generator=g).to(dtype)
    x = rows.double()
    x[:, :heads_width] = (rows[:, :heads_width].float() + bias.float()).to(dtype).double()  # (stored as a projection with a bias would be)
    q = x[:, : H * dk].reshape(n, H, dk).clone()
    k = x[:, H * dk : (H + G) * dk].reshape(n, G, dk).clone()
    v = x[:, (H + G) * dk : (H + G) * dk + G * dv].reshape(n, G, dv)
    eps = 1e-3

    def prepared(t, w):
        t = t.clone()
        head = t[..., :norm_dims]
        t[..., :norm_dims] = head / torch.sqrt((head * head).mean(-1, keepdim=True) + eps) * w.double()
        part = t[..., rot_off : rot_off + rot].clone()
        c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        if pairing == 0:
            a, b = part[..., 0::2], part[..., 1::2]
            part[..., 0::2], part[..., 1::2] = a * c - b * s, b * c + a * s
        else:
            a, b = part[..., : rot // 2], part[..., rot // 2 :]
            part = torch.cat([a * c - b * s, b * c + a * s], dim=-1)
        t[..., rot_off : rot_off + rot] = part
        return t

    factor = torch.tensor([1.0 + coef * math.log((p + 1) // every + 1) for p in positions], dtype=torch.float64)
    q_want = prepared(q, qw) * factor[:, None, None]
    k_want = prepared(k, kw)
    v_want = 0.7 * v + 0.3 * v_first.double().reshape(n, G, dv)

    d_rows = rows.to(dev)
    k_pages = torch.zeros((n_pages, G, page_size, dk), dtype=dtype, device=dev)
    v_pages = torch.zeros((n_pages, G, page_size, dv), dtype=dtype, device=dev)
    table = ops.rope_table(pos.to(dev), inv_freq.to(dev))
    ops.head_prepare(d_rows, H, G, dk, dv, bias=bias.to(dev), q_norm=qw.to(dev), k_norm=kw.to(dev), norm_dims=norm_dims, eps=eps, cos_sin=table,
                     rot_offset=rot_off, rot_dims=rot, pairing=pairing, positions=pos.to(dev), temp_coef=coef, temp_every=every,
                     v_first=v_first.to(dev), v_mix=lam.to(dev), k_pages=k_pages, v_pages=v_pages, slot_mapping=slots.to(dev),
                     page_size=page_size)
    out = d_rows.cpu().double()
    tol = _bf16_tol(dtype)
    torch.testing.assert_close(out[:, : H * dk].reshape(n, H, dk), q_want, **tol)
    torch.testing.assert_close(out[:, (H + G) * dk : (H + G) * dk + G * dv].reshape(n, G, dv), v_want, **tol)
    assert torch.equal(out[:, (H + G) * dk + G * dv :], x[:, (H + G) * dk + G * dv :])  # what follows the heads is left alone
    for t, slot in enumerate(slots.tolist()):
        torch.testing.assert_close(k_pages[slot // page_size, :, slot % page_size].cpu().double(), k_want[t], **tol)
        torch.testing.assert_close(v_pages[slot // page_size, :, slot % page_size].cpu().double(), v_want[t], **tol)
    # the factor steps exactly where floor((p + 1) / every) does
    assert factor[1] == factor[2] < factor[3] - 0.1 and factor[3] == factor[4] == factor[5] < factor[6] - 0.05 and factor[6] == factor[7]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_branch_norm_and_the_other_small_kernels(dtype):
    from torchllms_amd.kernels import ops

    dev = "cuda:0"
    g = torch.Generator().manual_seed(2)
    n, hidden = 37, 328
    stream = torch.randn((n, hidden), generator=g) * 3
    y = torch.randn((n, hidden), generator=g).to(dtype)
    w = torch.rand(hidden, generator=g) + 0.5
    want = stream.double() + y.double() / torch.sqrt((y.double() ** 2).mean(-1, keepdim=True) + 1e-5) * w.double()
    d_stream = stream.to(dev)
    rows = ops.branch_norm_add(d_stream, y.to(dev), w.to(dev), 1e-5)
    torch.testing.assert_close(d_stream.cpu().double(), want, rtol=1e-6, atol=1e-6)
    assert rows.dtype == dtype and torch.equal(rows.cpu(), d_stream.cpu().to(dtype))
    # a launch of many rows takes another form of the kernel than one of few: the same bits row by row
    many_stream, many_y = stream.repeat(20, 1).to(dev), y.repeat(20, 1).to(dev)
    ops.branch_norm_add(many_stream, many_y, w.to(dev), 1e-5)
    assert many_stream.shape[0] > 512 and torch.equal(many_stream[:n].cpu(), d_stream.cpu()) and torch.equal(many_stream[-n:].cpu(), d_stream.cpu())
    # a norm of some columns of a wider matrix, of gathered rows of a 32-bit matrix
    wide = torch.randn((n, hidden + 40), generator=g)
    idx = torch.tensor([5, 0, 36, 5], dtype=torch.int32)
    part = wide[:, 11 : 11 + hidden]
    got = ops.rmsnorm_columns(wide.to(dev)[:, 11 : 11 + hidden], w.to(dev), 1e-4, dtype, rows=idx.to(dev))
    sel = part[idx.long()].double()
    torch.testing.assert_close(got.cpu().double(), sel / torch.sqrt((sel ** 2).mean(-1, keepdim=True) + 1e-4) * w.double(), **_bf16_tol(dtype))
    # gates channel by channel and head by head (sizes that the 16-byte form takes, and sizes that it does not)
    for heads, d in ((6, 20), (8, 16)):
        x = torch.randn((n, heads * d), generator=g).to(dtype)
        gates = torch.randn((n, heads * d + heads), generator=g).to(dtype)
        by_channel = ops.sigmoid_gate_(x.to(dev).clone(), gates.to(dev)[:, : heads * d], per=1)
        torch.testing.assert_close(by_channel.cpu().double(), x.double() * torch.sigmoid(gates[:, : heads * d].double()), **_bf16_tol(dtype))
        by_head = ops.sigmoid_gate_(x.to(dev).clone(), gates.to(dev)[:, heads * d :], per=d)
        want_h = x.double().reshape(n, heads, d) * torch.sigmoid(gates[:, heads * d :].double())[:, :, None]
        torch.testing.assert_close(by_head.cpu().double().reshape(n, heads, d), want_h, **_bf16_tol(dtype))
    heads, d = 6, 20
    # packing and unpacking of heads
    a = torch.randn((heads, n, 9), generator=g).to(dtype)
    b = torch.randn((n, heads * 14 + 3), generator=g).to(dtype)
    packed = ops.pack_heads(a.to(dev), b.to(dev), 14, 10, 4).cpu().reshape(n, heads, 13)
    assert torch.equal(packed[:, :, :9], a.transpose(0, 1)) and torch.equal(packed[:, :, 9:], b[:, : heads * 14].reshape(n, heads, 14)[:, :, 10:])
    hg = torch.randn((n, heads), generator=g).to(dtype)
    un = ops.unpack_heads_gate(a.to(dev), hg.to(dev)).cpu().double().reshape(n, heads, 9)
    torch.testing.assert_close(un, a.double().transpose(0, 1) * torch.sigmoid(hg.double())[:, :, None], **_bf16_tol(dtype))
    z = torch.randn((n, 50), generator=g) * 30
    torch.testing.assert_close(ops.softcap_(z.to(dev).clone(), 20.0).cpu(), 20.0 * torch.tanh(z / 20.0), rtol=1e-5, atol=1e-5)


# ----------------------------------------------------------------------------- attention whose values lie in its keys
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
def test_one_far_key_stands_out_when_values_lie_inside_the_keys(form, dtype):
    """The plain attention kernel reading values out of the key rows, at an offset, on inputs in which one key far
    back (the first of all, one at a page's border, one in the middle, the query's own) has a score far above the
    hundreds of others: the output is that row's value channels.  All three launches of the kernel."""
    from torchllms_amd.kernels import ops

    dev = "cuda:0"
    H, d, dv, off, page = 3, 48, 20, 8, 16
    n = 700
    g = torch.Generator().manual_seed(3)
    k = torch.randn((n, 1, d), generator=g) * 0.2
    special = [0, 15, 16, 333, 639, 640, 699]
    directions = torch.nn.functional.normalize(torch.randn((len(special), d), generator=g), dim=-1)
    for i, j in enumerate(special):
        k[j, 0] += 5.0 * directions[i]  # its own direction: a query along it scores 40 there and a few elsewhere
    order = list(range(n // page + 1))
    random.Random(5).shuffle(order)
    pages, table = _paged(k.to(dtype).to(dev), page, order)
    k_all = k.to(dtype).double()[:, 0]  # as stored
    m = 40 if form == "tile" else 1  # (the tiled launch is for steps of at least 32 tokens)
    positions = torch.arange(n - m, n, dtype=torch.int32)
    tol = dict(rtol=3e-2, atol=3e-2) if dtype == torch.bfloat16 else dict(rtol=1e-4, atol=1e-4)
    for first in range(len(special)):
        targets = [(first + h) % len(special) for h in range(H)]  # head h looks for another key than its neighbours
        q = torch.cat([directions[i] * 8.0 for i in targets]).repeat(m, 1).to(dtype)
        args = (q.to(dev), H, 1, d, pages, pages, torch.zeros(m, dtype=torch.int32, device=dev), positions.to(dev), table, 0, 1.0)
        kw = dict(v_head_dim=dv, values_in_keys=True, value_offset=off)
        if form == "split":
            out = ops.attention_generic_split(*args, longest=n, **kw)
        else:
            out = ops.attention_generic(*args, **kw)
        out = out.cpu().double().reshape(m, H, dv)
        for h, i in enumerate(targets):
            for t in (0, m - 1):
                p = int(positions[t])
                w = torch.softmax(q.double()[t, h * d : (h + 1) * d] @ k_all[: p + 1].T, dim=-1)
                torch.testing.assert_close(out[t, h], w @ k_all[: p + 1, off : off + dv], **tol)
                if special[i] <= p:
                    assert float(w[special[i]]) > 0.99  # the inputs do single that key out
                    torch.testing.assert_close(out[t, h], k_all[special[i], off : off + dv], rtol=0.05, atol=0.05)


def test_float32_bits_do_not_depend_on_the_rows_of_a_step(tmp_path):
    """A prompt of more rows than the kernels' forms for few rows take, whole, against the same tokens in a long
    portion, a short one and single tokens: kernels that have a form for few rows and one for many add alike."""
    from torchllms_amd.engine import Engine, StepEntry

    folder = models.make_folder(tmp_path / "m", models.CONFIGS["A"], seed=2)
    cfg, _ = models.read_folder(folder)
    tokens = random_tokens(660, cfg["vocab"], 4)
    engine = Engine.from_folder(folder, dtype="float32", page_size=16, num_pages=96, max_seqs=2)
    engine.admit("whole")
    whole = engine.step([StepEntry("whole", tokens, list(range(len(tokens))))]).cpu()
    engine.admit("cut")
    rows, at = [], 0
    for n in [560, 70] + [1] * 30:
        rows.append(engine.step([StepEntry("cut", tokens[at : at + n], list(range(n)))]).cpu())
        at += n
    assert at == len(tokens)
    assert torch.equal(torch.cat(rows), whole)


# ----------------------------------------------------------------------------- long decoding, generation, drawn configurations
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_from_recorded_steps(tmp_path, dtype):
    """A short prompt and 300 tokens one by one, two requests side by side: the decode steps are recorded as
    graphs after a few and replayed; the query factor steps many times on the way and the first keys stay visible."""
    from torchllms_amd.engine import Engine, StepEntry

    folder = models.make_folder(tmp_path / "m", models.CONFIGS["A"], seed=8)
    cfg, weights = models.read_folder(folder)
    requests = {"a": random_tokens(310, cfg["vocab"], 1), "b": random_tokens(325, cfg["vocab"], 2)}
    truth, scale = truth_of(cfg, weights, requests)
    engine = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=48, max_seqs=2)
    assert engine.graphs is not None
    heads = {"a": 10, "b": 25}
    for rid, toks in requests.items():
        engine.admit(rid)
        engine.step([StepEntry(rid, toks[: heads[rid]], [])])
    tol = FP32_TOL if dtype == "float32" else bfloat16_bounds(cfg, weights, requests, truth, scale)[0]
    worst = 0.0
    for i in range(300):
        entries = [StepEntry(rid, [requests[rid][heads[rid] + i]], [0]) for rid in ("a", "b")]
        logits = engine.step(entries).cpu()
        for row, rid in zip(logits, ("a", "b")):
            worst = max(worst, distance(row, truth[rid][heads[rid] + i], scale))
    assert any(g.replays > 100 for g in engine.graphs.graphs.values())
    assert worst < tol, worst


def test_greedy_generation_through_the_entry_point(tmp_path):
    """``LLM.generate``: the scheduler admits, cuts prompts into portions under a small token budget, decodes
    everybody together and frees; the tokens are the plain model's."""
    from torchllms_amd.inference import LLM

    folder = models.make_folder(tmp_path / "m", models.CONFIGS["B"], seed=4)
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
    llm16 = LLM(str(folder), precision="bfloat16", max_len=128, max_bsz=3, page_size=8)
    for p, r in zip(prompts, llm16.generate(prompt_token_ids=prompts, temperature=0.0, max_new_tokens=4)):
        logits = plain.forward(cfg, w64, p)[-1]
        assert logits[r.token_ids[0]] >= logits.max() - 0.05 * float(logits.std())


def test_a_preempted_request_is_computed_again_with_the_same_tokens(tmp_path):
    """Too few pages for four requests: the scheduler takes the youngest off, gives its pages and its slot away and
    later computes it again from its prompt and what it had generated (keys, latent rows and mixed values land in
    other pages): the sampled tokens are those of the run with room for everybody."""
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

    from torchllms_amd.config.vobolorn import VobolornConfig
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
    written = write_model_folder(tmp_path / "written", VobolornConfig.from_dict(models.CONFIGS["B"]), seed=7, dtype=torch.float32)
    cfg, weights = models.read_folder(written)
    w64 = {k: v.double() for k, v in weights.items()}
    toks = list(prompt)
    for _ in range(6):
        toks.append(int(plain.forward(cfg, w64, toks)[-1].argmax()))
    assert got == toks[len(prompt):]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_program(tmp_path, dtype):
    """``bin/trace_run`` as a process: steps in, logits files out, the plain model's values; the pool is made for
    the live requests only, so pages and slots of requests that ended are used again."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    root = Path(__file__).resolve().parent.parent
    folder = models.make_folder(tmp_path / "m", models.CONFIGS["A"], seed=6)
    cfg, weights = models.read_folder(folder)
    requests = {"x": random_tokens(50, cfg["vocab"], 1), "y": random_tokens(90, cfg["vocab"], 2), "z": random_tokens(20, cfg["vocab"], 3),
                "u": random_tokens(70, cfg["vocab"], 4), "v": random_tokens(33, cfg["vocab"], 5)}
    truth, scale = truth_of(cfg, weights, requests)
    tol = FP32_TOL if dtype == "float32" else bfloat16_bounds(cfg, weights, requests, truth, scale)[0]
    steps = schedules.mixed(requests, max_live=2)
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, str(root / "bin" / "trace_run"), "--model", str(folder), "--dtype", dtype, "--out", str(out),
         "--max-tokens", str(schedules.max_live_tokens(steps))],
        input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600,
    )
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done ")] == [f"done {i}" for i in range(len(steps))]
    for step, rows in zip(steps, schedules.positions_of(steps)):
        if not rows:  # (a step in which nothing is wanted writes no file)
            assert not (out / f"{step['step']}.f32").exists()
            continue
        got = torch.from_numpy(np.fromfile(out / f"{step['step']}.f32", dtype="<f4").reshape(len(rows), -1))
        for row, (rid, pos) in zip(got, rows):
            assert distance(row, truth[rid][pos], scale) < tol


def drawn_config(seed: int) -> dict:
    """A configuration drawn from a seed: the order of layers, every size and constant (sizes that the matrix-core
    attention kernels take among them, for keys and values alike and for the latent layer's rows)."""
    rng = random.Random(seed)
    width = rng.choice([40, 64, 72, 96, 160])
    mixing = None  # (kv_heads, vdim) that the mixing layers share
    layers = []
    for _ in range(rng.randint(1, 5)):
        kind = rng.choice(["attention", "attention_2", "latent_attention"])
        ff = rng.choice([None, 40, 88, 136])
        if kind == "latent_attention":
            kv_rank, rot = rng.choice([(10, 2), (32, 6), (68, 16), (48, 16), (96, 32), (130, 0), (192, 64), (264, 8)])
            layers.append(models.layer(models.latent(rng.randint(1, 9), rng.choice([8, 12, 32, 64]), rot, rng.choice([8, 20, 36, 64]),
                                                     rng.choice([8, 24, 48]), kv_rank, rng.uniform(0.1, 0.5),
                                                     base=rng.choice([10.0, 10000.0, 500000.0])), ff=ff))
            continue
        mix = rng.random() < 0.6
        kv = rng.choice([1, 2, 3])
        dim = rng.choice([8, 18, 32, 64, 96, 128])
        vdim = rng.choice([8, 18, 32, dim, dim])
        if mix:
            if mixing is None:
                mixing = (kv, vdim)
            kv, vdim = mixing
        heads = kv * rng.choice([1, 2, 5, 8])
        q_temp = (rng.uniform(0.1, 1.0), rng.choice([1, 3, 17, 64])) if kind == "attention_2" else None
        layers.append(models.layer(models.grouped(kind, heads, kv, dim, vdim, rng.uniform(0.2, 0.8) * (32 / dim) ** 0.5,
                                                  q_temp=q_temp, v_mix=mix), ff=ff))
    return models.model(rng.choice([50, 97, 160, 515]), width, rng.choice([1e-5, 1e-6, 1e-3]), layers,
                        softcap=rng.choice([None, 5.0, 30.0]))


@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_from_seeds(tmp_path, seed):
    """A prompt whole and then cut at random beside a second request, 32-bit against the twin and bit for bit against
    itself, bfloat16 within rounding."""
    from torchllms_amd.engine import Engine, StepEntry

    cfg_dict = drawn_config(seed)
    folder = models.make_folder(tmp_path / "m", cfg_dict, seed=seed)
    cfg, weights = models.read_folder(folder)
    rng = random.Random(100 + seed)
    requests = {"a": random_tokens(rng.randint(60, 140), cfg["vocab"], seed), "b": random_tokens(rng.randint(20, 60), cfg["vocab"], seed + 50)}
    truth, scale = truth_of(cfg, weights, requests)
    page = rng.choice([4, 8, 16, 16])
    for dtype, tol in (("float32", float32_bound(cfg, weights, requests, truth, scale)),
                       ("bfloat16", bfloat16_bounds(cfg, weights, requests, truth, scale)[0])):
        engine = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=-(-400 // page), max_seqs=3)
        engine.admit("w")
        whole = engine.step([StepEntry("w", requests["a"], list(range(len(requests["a"]))))]).cpu()
        engine.free("w")
        engine.admit("a")
        engine.admit("b")
        at = {"a": 0, "b": 0}
        got = {"a": [], "b": []}
        while any(at[r] < len(requests[r]) for r in at):
            entries = []
            for r in ("b", "a"):
                left = len(requests[r]) - at[r]
                if left and rng.random() < 0.8:
                    n = min(left, rng.choice([1, 1, 2, 3, 9, 40]))
                    entries.append(StepEntry(r, requests[r][at[r] : at[r] + n], list(range(n))))
                    at[r] += n
            if not entries:
                continue
            logits = engine.step(entries).cpu()
            row = 0
            for e in entries:
                got[e.rid].append(logits[row : row + len(e.tokens)])
                row += len(e.tokens)
        cut = {r: torch.cat(got[r]) for r in got}
        for r in ("a", "b"):
            worst = max(distance(cut[r][i], truth[r][i], scale) for i in range(len(requests[r])))
            assert worst < tol, f"seed {seed} {dtype} request {r}: distance {worst}; {cfg_dict}"
        if dtype == "float32":
            assert torch.equal(whole, cut["a"]), f"seed {seed}: {cfg_dict}"
