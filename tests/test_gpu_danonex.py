"""The Danonex model through the engine's step function, cache and kernels against the plain
implementation (tests/plain/danonex_plain.py, float64 on the same weights).

Per model and precision one replayer runs the same requests whole, decoded token by token from
the first token on, in portions of several sizes down to two tokens, and mixed: unequal requests
side by side in a pool and in state slots so small that pages and slots are given back and used
again.  Every logit is compared with the plain one.  Greedy generation goes through the engine's
own entry point and scheduler, and through `bin/trace_run` as a program.
"""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import danonex_models as M
from tests import helpers
from tests.plain import danonex_plain as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = (150, 37, 90, 1)
PORTIONS = (7, 2, 5, 3, 2, 11, 4, 2, 9, 17, 33)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("danonex")
    return {name: M.make_folder(tmp, name) for name in M.CONFIGS}


_PLAIN = {}


def plain_logits(folders, name, length):
    key = (name, length)
    if key not in _PLAIN:
        cfg, weights = M.read_folder(folders[name])
        _PLAIN[key] = plain.forward(weights, cfg, M.tokens_for(name, length), torch.float64)
    return _PLAIN[key]


def rounding_alone(folders, name, tokens, want):
    """(largest, root-mean-square) error of the plain implementation when its products' operands and
    results are rounded to bfloat16 and nothing else changes: what reduced precision costs this model
    on these tokens, whatever the kernels."""
    cfg, weights = M.read_folder(folders[name])
    worst = rms = 0.0
    plain.STORAGE = torch.bfloat16
    try:
        for trial in range(4):  # the products' sums as they are, and in three other orders of adding
            plain.JITTER = (torch.Generator().manual_seed(trial), 3e-4) if trial else None
            diff = plain.forward(weights, cfg, tokens, torch.float64) - want
            worst, rms = max(worst, float(diff.abs().max())), max(rms, float(diff.pow(2).mean().sqrt()))
    finally:
        plain.STORAGE = plain.JITTER = None
    return worst, rms


_ROUNDING = {}


def rounding_of(folders, name, length):
    if (name, length) not in _ROUNDING:
        _ROUNDING[name, length] = rounding_alone(folders, name, M.tokens_for(name, length), plain_logits(folders, name, length))
    return _ROUNDING[name, length]


def check(got, want, dtype, what, rounding=None):
    """float32: a few hundred roundings relative to the largest logit.  bfloat16: these models are made
    to be touchy (peaked attention, norms right after small sums), so the measure is what rounding alone
    does to the plain implementation on the same tokens (`rounding` = its largest and root-mean-square
    error): the engine may be off by three times that plus a unit in the last place of the largest logit."""
    got, want = torch.as_tensor(got).double(), torch.as_tensor(want).double()
    top = float(want.abs().max())
    worst = float((got - want).abs().max())
    if dtype == "float32":
        assert worst <= 1e-4 * top, f"{what}: worst logit error {worst:.3e} > {1e-4 * top:.3e}"
        return worst
    if rounding is None:
        return helpers.check_logits(got, want, dtype, "wide", what)
    bound = 3.0 * rounding[0] + helpers.bf16_ulp(want)
    assert worst <= bound, f"{what}: worst logit error {worst:.3e} > {bound:.3e} (rounding alone {rounding[0]:.3e})"
    rms = float((got - want).pow(2).mean().sqrt())
    if got.shape[0] >= 16:
        assert rms <= 2.0 * rounding[1] + 2.0 ** -9 * top, f"{what}: rms logit error {rms:.3e} (rounding alone {rounding[1]:.3e})"
    return worst


def replayer(folders, name, dtype, max_tokens, max_live=4, block_size=16):
    from paged_attention_engine_amd.engine.trace import TraceReplayer

    return TraceReplayer(folders[name], dtype, max_tokens, block_size, max_live)


def run_alone(rp, rid, tokens, cuts, want_all=True):
    """Feed `tokens` as one request in portions of the sizes `cuts` (cycled); returns [T, vocab]."""
    rows, p, i = [], 0, 0
    while p < len(tokens):
        n = min(cuts[i % len(cuts)], len(tokens) - p)
        i += 1
        out = rp.step({"step": 0, "entries": [{"id": rid, "tokens": tokens[p:p + n], "want": list(range(n))}],
                       "end": [rid] if p + n == len(tokens) else []})
        rows.append(torch.from_numpy(out.copy()))
        p += n
    return torch.cat(rows)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(M.CONFIGS))
def test_whole_decoded_and_in_portions(folders, name, dtype):
    """A prompt whole, token by token from its first token on (which is prefill against decoding,
    and a long decode), and in portions of changing sizes: all against the plain logits, and in
    float32 the three against each other to a few roundings."""
    rp = replayer(folders, name, dtype, 256)
    for length in LENGTHS[:3]:
        tokens = M.tokens_for(name, length)
        want = plain_logits(folders, name, length)
        rounding = rounding_of(folders, name, length) if dtype == "bfloat16" else None
        whole = run_alone(rp, "w", tokens, (length,))
        check(whole, want, dtype, f"{name} {dtype} whole {length}", rounding)
        single = run_alone(rp, "d", tokens, (1,))
        check(single, want, dtype, f"{name} {dtype} token by token {length}", rounding)
        for first in (0, 4):
            cut = run_alone(rp, "c", tokens, PORTIONS[first:] + PORTIONS[:first])
            check(cut, want, dtype, f"{name} {dtype} portions {length}", rounding)
        cut = run_alone(rp, "c2", tokens, (2,))
        check(cut, want, dtype, f"{name} {dtype} portions of two {length}", rounding)
        if dtype == "float32":
            top = float(want.abs().max())
            assert float((whole - single).abs().max()) <= 2e-5 * top
            assert float((whole - cut).abs().max()) <= 2e-5 * top
    assert rp.cache.slots.num_free == 4 and all(g.allocator.num_free == g.allocator.num_blocks for g in rp.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q", "R"])
def test_the_first_tokens_of_a_sequence(folders, name, dtype):
    """One token, two, and as many as the longest convolution has taps, each as a request of its own."""
    rp = replayer(folders, name, dtype, 64)
    for length in (1, 2, 3, 4, 5):
        cfg, weights = M.read_folder(folders[name])
        tokens = M.tokens_for(name, length, salt=7)
        want = plain.forward(weights, cfg, tokens, torch.float64)
        rounding = rounding_alone(folders, name, tokens, want) if dtype == "bfloat16" else None
        check(run_alone(rp, "f", tokens, (length,)), want, dtype, f"{name} first {length} whole", rounding)
        check(run_alone(rp, "g", tokens, (1,)), want, dtype, f"{name} first {length} one by one", rounding)


def mixed_schedule(lengths):
    """Steps of (request index, count): requests arrive staggered, run a portion a step and then
    single tokens beside the others' portions; at most four are live; every request runs twice."""
    order = [i for _ in range(2) for i in range(len(lengths))]
    steps, live, done_of, arrivals = [], {}, {}, list(enumerate(order))
    tick = 0
    while arrivals or live:
        if arrivals and len(live) < 4 and tick % 2 == 0:
            rid, which = arrivals.pop(0)
            live[rid] = [which, 0]
        step = []
        for rid, (which, at) in list(live.items()):
            left = lengths[which] - at
            tail = min(12, lengths[which] // 2)
            n = 1 if left <= tail else min(PORTIONS[(tick + rid) % len(PORTIONS)], left - tail)
            if (tick + rid) % 5 == 4 and left > 1:
                continue  # a request is left out of a step and goes on later
            step.append((rid, which, at, n))
            live[rid][1] = at + n
            if at + n == lengths[which]:
                del live[rid]
        if step:
            steps.append(step)
        tick += 1
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(M.CONFIGS))
def test_unequal_requests_side_by_side_with_pages_and_slots_used_again(folders, name, dtype):
    lengths = LENGTHS
    tokens = [M.tokens_for(name, n) for n in lengths]
    want = [plain_logits(folders, name, n) for n in lengths]
    rounding = [rounding_of(folders, name, n) if dtype == "bfloat16" else None for n in lengths]
    steps = mixed_schedule(lengths)
    # the pool holds what the four longest live requests need and no more, so pages are used again
    rp = replayer(folders, name, dtype, sum(-(-n // 64) * 64 for n in lengths))
    seen_slots, worst = set(), 0.0
    for step in steps:
        record = {"step": 0, "entries": [], "end": []}
        for rid, which, at, n in step:
            record["entries"].append({"id": f"r{rid}", "tokens": tokens[which][at:at + n], "want": list(range(n))})
            if at + n == lengths[which]:
                record["end"].append(f"r{rid}")
        out = torch.from_numpy(rp.step(record).copy())
        seen_slots.update(rp.cache.slots.held().values())
        row = 0
        for rid, which, at, n in step:
            worst = max(worst, check(out[row:row + n], want[which][at:at + n], dtype,
                                     f"{name} {dtype} request {rid} rows {at}..{at + n}", rounding[which]))
            row += n
    assert len(steps) > 30 and max(len(s) for s in steps) == 4
    assert rp.cache.slots.num_free == 4
    if dtype == "float32" and rp.runner.use_graphs:
        assert rp.runner.graph_replays > 0  # steps of single tokens ran as recorded graphs


def test_recorded_steps_give_the_eager_steps_logits(folders):
    """Steps of single tokens replay as HIP graphs; the same steps launched kernel by kernel give the same bits."""
    from paged_attention_engine_amd.engine.step import StepRunner

    tokens = M.tokens_for("P", 60)
    outs = []
    for graphs in (True, False):
        rp = replayer(folders, "P", "float32", 128)
        rp.runner = StepRunner(rp.model, rp.cache, use_graphs=graphs)
        outs.append(run_alone(rp, "a", tokens, (20,) + (1,) * 40))
        if graphs:
            assert rp.runner.graph_replays >= 39
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "S"])
def test_greedy_generation_through_the_entry_point(folders, name, dtype):
    import paged_attention_engine_amd as pae

    cfg, weights = M.read_folder(folders[name])
    prompt = M.tokens_for(name, 21, salt=3)
    want_tokens, want_logits = plain.greedy_generate(weights, cfg, prompt, 12, torch.float64)
    engine = pae.Engine(folders[name], dtype=dtype, block_size=16, num_blocks=8, max_num_seqs=2)
    got = engine.generate(prompt, 12)
    same = 0
    while same < 12 and got.token_ids[same] == want_tokens[same]:
        same += 1
    rows = min(same + 1, 12)
    check(got.step_logits[:rows].cpu(), want_logits[:rows], dtype, f"{name} {dtype} generation")
    if dtype == "float32":
        assert list(got.token_ids) == want_tokens
    else:  # a different token only where the plain logits nearly tie
        top2 = want_logits.topk(2, dim=-1).values
        assert same == 12 or float(top2[same, 0] - top2[same, 1]) <= 2 * helpers.bf16_atol(want_logits, "wide")


def test_requests_through_the_scheduler_with_few_pages(folders):
    """Several requests through the scheduler in a pool that forces waiting and portions; every
    request's tokens are those it generates alone."""
    import paged_attention_engine_amd as pae

    prompts = [M.tokens_for("P", n, salt=9) for n in (33, 5, 70, 18, 41)]
    alone = []
    for prompt in prompts:
        engine = pae.Engine(folders["P"], dtype="float32", block_size=16, num_blocks=16, max_num_seqs=1)
        alone.append(list(engine.generate(prompt, 10).token_ids))
    engine = pae.Engine(folders["P"], dtype="float32", block_size=16, num_blocks=14, max_num_seqs=3,
                        max_num_batched_tokens=24)
    for i, prompt in enumerate(prompts):
        assert engine.add_request(pae.Request(f"r{i}", tuple(prompt), max_new_tokens=10))
    done = engine.run_to_completion()
    assert [list(done[f"r{i}"]) for i in range(len(prompts))] == alone


def test_the_program_replays_a_trace(folders, tmp_path):
    """bin/trace_run as a program: steps on standard input, logits in files, `done` lines."""
    tokens = M.tokens_for("Q", 37)
    want = plain_logits(folders, "Q", 37)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": tokens[:20], "want": [0, 19]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": tokens[20:22], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": tokens[22:], "want": [14]}], "end": ["a"]}]
    out = tmp_path / "logits"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders["Q"], "--dtype",
                           "float32", "--out", str(out), "--max-tokens", "64"],
                          input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [line for line in proc.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1", "done 2"]
    assert not (out / "1.f32").exists()
    first = np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1)
    last = np.fromfile(out / "2.f32", dtype="<f4").reshape(1, -1)
    check(first, want[[0, 19]], "float32", "trace_run step 0")
    check(last, want[[36]], "float32", "trace_run step 2")
