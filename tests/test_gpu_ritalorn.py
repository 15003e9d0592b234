"""The Ritalorn model through the engine's step function, cache and kernels against the plain
implementation (tests/plain/ritalorn_plain.py, float64 on the same weights).

Per model and precision one replayer runs the same requests whole, decoded token by token from
the first token on, in portions of several sizes down to two tokens, and mixed: unequal requests
side by side in a pool and in state slots so small that pages and slots are given back and used
again.  Every logit is compared with the plain one, and so is the stream after every layer.  Greedy
generation goes through the engine's own entry point and scheduler, and through `bin/trace_run`.
The prompts are longer than every window and chunk of the models but two, so that keys just inside and
just outside every edge are asked for in prompts, in portions and by single tokens.
"""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import helpers
from tests import ritalorn_models as M
from tests.plain import ritalorn_plain as plain
from tests.test_gpu_danonex import PORTIONS, mixed_schedule, run_alone

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = (150, 37, 90, 1)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("ritalorn")
    return {name: M.make_folder(tmp, name) for name in M.CONFIGS}


_PLAIN, _ROUNDING = {}, {}


def plain_logits(folders, name, length):
    key = (name, length)
    if key not in _PLAIN:
        cfg, weights = M.read_folder(folders[name])
        _PLAIN[key] = plain.forward(weights, cfg, M.tokens_for(name, length), torch.float64)
    return _PLAIN[key]


def rounding_alone(folders, name, tokens, want):
    """(largest, root-mean-square) error of the plain implementation when its products' operands and
    results are rounded to bfloat16 and nothing else changes, the sums as they are and moved a little."""
    cfg, weights = M.read_folder(folders[name])
    worst = rms = 0.0
    plain.STORAGE = torch.bfloat16
    try:
        for trial in range(4):
            plain.JITTER = (torch.Generator().manual_seed(trial), 3e-4) if trial else None
            diff = plain.forward(weights, cfg, tokens, torch.float64) - want
            worst, rms = max(worst, float(diff.abs().max())), max(rms, float(diff.pow(2).mean().sqrt()))
    finally:
        plain.STORAGE = plain.JITTER = None
    return worst, rms


def rounding_of(folders, name, length):
    if (name, length) not in _ROUNDING:
        _ROUNDING[name, length] = rounding_alone(folders, name, M.tokens_for(name, length), plain_logits(folders, name, length))
    return _ROUNDING[name, length]


def check(got, want, dtype, what, rounding=None):
    """float32: 1e-4 of the largest logit.  bfloat16: three times what rounding alone does to the plain
    implementation on the same tokens, plus a unit in the last place of the largest logit."""
    got, want = torch.as_tensor(got).double(), torch.as_tensor(want).double()
    top = float(want.abs().max())
    worst = float((got - want).abs().max())
    if dtype == "float32":
        assert worst <= 1e-4 * top, f"{what}: worst logit error {worst:.3e} > {1e-4 * top:.3e}"
        return worst
    bound = 3.0 * rounding[0] + helpers.bf16_ulp(want)
    assert worst <= bound, f"{what}: worst logit error {worst:.3e} > {bound:.3e} (rounding alone {rounding[0]:.3e})"
    rms = float((got - want).pow(2).mean().sqrt())
    if got.shape[0] >= 16:
        assert rms <= 2.0 * rounding[1] + 2.0 ** -9 * top, f"{what}: rms logit error {rms:.3e} (rounding alone {rounding[1]:.3e})"
    return worst


def replayer(folders, name, dtype, max_tokens, max_live=4, block_size=16):
    from paged_attention_engine_amd.engine.trace import TraceReplayer

    return TraceReplayer(folders[name], dtype, max_tokens, block_size, max_live)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(M.CONFIGS))
def test_whole_decoded_and_in_portions(folders, name, dtype):
    """A prompt whole, token by token from its first token on (prefill against decoding, and a long
    decode that walks over every window's and chunk's edge), and in portions of changing sizes."""
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


@pytest.mark.parametrize("name", ["A", "C"])
def test_the_stream_after_every_layer(folders, name):
    """The sum of the stream's copies after every layer, float32, whole prompt and token by token."""
    from paged_attention_engine_amd.engine.step import StepRunner

    rp = replayer(folders, name, "float32", 128)
    rp.runner = StepRunner(rp.model, rp.cache, use_graphs=False)  # the tap reads the stream on the host
    cfg, weights = M.read_folder(folders[name])
    tokens = M.tokens_for(name, 70, salt=2)
    _, want = plain.forward(weights, cfg, tokens, torch.float64, keep_layers=True)
    copies = int(cfg["streams"])
    seen = []

    def tap(index, stream):
        x = stream.residual.view(stream.residual.shape[0], copies, -1).double()
        y = stream.pending.double().sum(0) if stream.pending.dim() == 3 else stream.pending.double()
        y = y * stream.join.scale.double()
        x = torch.einsum("st,bsh->bth", stream.join.mix.double(), x) + stream.join.out.double()[None, :, None] * y[:, None, :]
        seen.append((index, x.sum(1).cpu()))

    rp.model.residual_tap = tap
    try:
        run_alone(rp, "w", tokens, (len(tokens),))
        for index, got in seen:
            top = float(want[index].abs().max())
            assert float((got - want[index]).abs().max()) <= 2e-5 * top, f"{name}: the stream after layer {index}"
        del seen[:]
        run_alone(rp, "d", tokens, (64,) + (1,) * 6)
        last = {index: got for index, got in seen}  # the last token's rows, decoded alone
        for index, got in last.items():
            top = float(want[index].abs().max())
            assert float((got[0] - want[index][-1]).abs().max()) <= 2e-5 * top, f"{name}: decoded, after layer {index}"
    finally:
        rp.model.residual_tap = None


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "E"])
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
    for step in steps:
        record = {"step": 0, "entries": [], "end": []}
        for rid, which, at, n in step:
            record["entries"].append({"id": f"r{rid}", "tokens": tokens[which][at:at + n], "want": list(range(n))})
            if at + n == lengths[which]:
                record["end"].append(f"r{rid}")
        out = torch.from_numpy(rp.step(record).copy())
        row = 0
        for rid, which, at, n in step:
            check(out[row:row + n], want[which][at:at + n], dtype, f"{name} {dtype} request {rid} rows {at}..{at + n}",
                  rounding[which])
            row += n
    assert len(steps) > 30 and max(len(s) for s in steps) == 4
    assert rp.cache.slots.num_free == 4
    if dtype == "float32" and rp.runner.use_graphs:
        assert rp.runner.graph_replays > 0  # steps of single tokens ran as recorded graphs


def test_a_slot_that_held_another_request_starts_from_nothing(folders):
    """With one state slot every request gets the slot the one before left: the convolutions' remembered
    inputs of the old request must not reach the new one's first tokens."""
    rp = replayer(folders, "A", "float32", 128, max_live=1)
    for salt in (1, 2, 3):
        tokens = M.tokens_for("A", 30, salt=salt)
        cfg, weights = M.read_folder(folders["A"])
        want = plain.forward(weights, cfg, tokens, torch.float64)
        check(run_alone(rp, f"s{salt}", tokens, (3, 1, 1, 9)), want, "float32", f"slot used again, request {salt}")


def test_recorded_steps_give_the_eager_steps_logits(folders):
    """Steps of single tokens replay as HIP graphs; the same steps launched kernel by kernel give the same bits."""
    from paged_attention_engine_amd.engine.step import StepRunner

    tokens = M.tokens_for("A", 60)
    outs = []
    for graphs in (True, False):
        rp = replayer(folders, "A", "float32", 128)
        rp.runner = StepRunner(rp.model, rp.cache, use_graphs=graphs)
        outs.append(run_alone(rp, "a", tokens, (20,) + (1,) * 40))
        if graphs:
            assert rp.runner.graph_replays >= 39
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
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
    if dtype == "float32":
        check(got.step_logits[:rows].cpu(), want_logits[:rows], dtype, f"{name} {dtype} generation")
        assert list(got.token_ids) == want_tokens
    else:  # a different token only where the plain logits nearly tie
        helpers.check_logits(got.step_logits[:rows].cpu(), want_logits[:rows], dtype, "wide", f"{name} {dtype} generation")
        top2 = want_logits.topk(2, dim=-1).values
        assert same == 12 or float(top2[same, 0] - top2[same, 1]) <= 2 * helpers.bf16_atol(want_logits, "wide")


def test_requests_through_the_scheduler_with_few_pages(folders):
    """Several requests through the scheduler in a pool that forces waiting and portions; every
    request's tokens are those it generates alone."""
    import paged_attention_engine_amd as pae

    prompts = [M.tokens_for("A", n, salt=9) for n in (33, 5, 70, 18, 41)]
    alone = []
    for prompt in prompts:
        engine = pae.Engine(folders["A"], dtype="float32", block_size=16, num_blocks=16, max_num_seqs=1)
        alone.append(list(engine.generate(prompt, 10).token_ids))
    engine = pae.Engine(folders["A"], dtype="float32", block_size=16, num_blocks=14, max_num_seqs=3,
                        max_num_batched_tokens=24)
    for i, prompt in enumerate(prompts):
        assert engine.add_request(pae.Request(f"r{i}", tuple(prompt), max_new_tokens=10))
    done = engine.run_to_completion()
    assert [list(done[f"r{i}"]) for i in range(len(prompts))] == alone


def test_the_program_replays_a_trace(folders, tmp_path):
    """bin/trace_run as a program: steps on standard input, logits in files, `done` lines."""
    tokens = M.tokens_for("B", 37)
    want = plain_logits(folders, "B", 37)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": tokens[:20], "want": [0, 19]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": tokens[20:22], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": tokens[22:], "want": [14]}], "end": ["a"]}]
    out = tmp_path / "logits"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders["B"], "--dtype",
                           "float32", "--out", str(out), "--max-tokens", "64"],
                          input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [line for line in proc.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1", "done 2"]
    assert not (out / "1.f32").exists()
    first = np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1)
    last = np.fromfile(out / "2.f32", dtype="<f4").reshape(1, -1)
    check(first, want[[0, 19]], "float32", "trace_run step 0")
    check(last, want[[36]], "float32", "trace_run step 2")
