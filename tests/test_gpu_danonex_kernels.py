"""The kernels behind the Danonex mixers, each against the plain function of the same mechanism
(tests/plain/danonex_plain.py, float64), on inputs made so that a fault shows: one far key whose
score stands out among hundreds, keys on both sides of page borders, sinks that take most of a
softmax or none of it, a cap that bites, rotations over part of a head, states carried over
steps cut at every place.
"""

import math

import pytest
import torch

from tests.plain import danonex_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def _K():
    from paged_attention_engine_amd.kernels import lib
    return lib


def scattered_table(num_pages: int, spare: int, seed: int):
    gen = torch.Generator().manual_seed(seed)
    return torch.randperm(num_pages + spare, generator=gen)[:num_pages].to(torch.int32)


def fill_cache(k, v, table, bs, dtype, spare=3):
    """k [T, G, D], v [T, G, V] into pools laid out as the attention kernels read them."""
    T, G, D = k.shape
    V = v.shape[2]
    pages = table.numel() + spare
    kc = torch.zeros(pages, G, bs, D, dtype=dtype)
    vc = torch.zeros(pages, G, V, bs, dtype=dtype)
    for t in range(T):
        kc[table[t // bs], :, t % bs] = k[t].to(dtype)
        vc[table[t // bs], :, :, t % bs] = v[t].to(dtype)
    return kc.to(DEV), vc.to(DEV)


def attend(out, q, kc, vc, positions, tok_seq, tables, runs, H, G, D, V, scale, window, cap, sinks):
    """The product's own choice of kernels for a step whose sequences are `runs` = (table row, first
    flat row, rows, tokens held before): work lists as the attention part builds them, then `attend_paged`."""
    from paged_attention_engine_amd.kernels import lib
    from paged_attention_engine_amd.parts import StepShape
    from paged_attention_engine_amd.parts.attention import attend_paged, attention_work_lists

    bs = kc.shape[2]
    work = None
    if V == D and lib.mfma_attention_supported(q.dtype, H, G, D, bs):
        assert [r[0] for r in runs] == list(range(len(runs)))
        shape = StepShape(tuple(range(len(runs))), tuple(r[1] for r in runs), tuple(r[2] for r in runs),
                          tuple(r[3] for r in runs), bs)
        work = {}
        for name, (flat, width) in attention_work_lists(shape).items():
            work[name] = torch.tensor(flat, dtype=torch.int32, device=DEV).view(-1, width)
    attend_paged(out, q, kc, vc, positions, tok_seq, tables, work, H, G, D, V, scale, window, cap, sinks)
    return work is not None


def tolerance(dtype, want):
    return (2e-5 if dtype == torch.float32 else 2.5e-2) * float(want.abs().max())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,V,cap,bs", [(4, 2, 32, 32, 25.0, 16), (6, 2, 64, 64, 0.0, 16), (3, 1, 48, 80, 6.0, 16),
                                            (2, 1, 160, 160, 30.0, 32), (5, 5, 20, 12, 0.0, 8)])
def test_attention_with_cap_sinks_and_value_width(dtype, H, G, D, V, cap, bs):
    """A prompt of 700 tokens in one step, then single tokens: every query against the plain softmax.
    Query 699 and key 5 are scaled so that their score stands out (a far key among hundreds), queries
    at page borders look at keys just before and after the border, head 0's sink takes most of the
    softmax, the last head's none."""
    K = _K()
    T = 700
    gen = torch.Generator().manual_seed(D * 7 + V)
    q = torch.randn(T, H, D, generator=gen, dtype=torch.float64) * 0.7
    k = torch.randn(T, G, D, generator=gen, dtype=torch.float64) * 0.7
    v = torch.randn(T, G, V, generator=gen, dtype=torch.float64)
    direction = torch.randn(D, generator=gen, dtype=torch.float64)
    direction /= direction.norm()
    k[5] = 4.0 * direction
    q[699] = 4.0 * direction
    for border in (bs * 9, bs * 20):   # the key just before a border and the one just after it
        k[border - 1] = 3.0 * direction
        k[border] = -3.0 * direction
        q[border] = 3.0 * direction
        q[border + 1] = 3.0 * direction
    sinks = torch.linspace(6.0, -9.0, H, dtype=torch.float64)
    scale = 1.3 / math.sqrt(D) * 4
    # what the kernel sees: operands rounded to its storage type
    qr, kr, vr = (x.to(dtype).double() for x in (q, k, v))
    want = plain.attend(qr, kr, vr, scale, cap or None, sinks).reshape(T, H * V)
    table = scattered_table(-(-T // bs), 3, seed=D)
    kc, vc = fill_cache(k, v, table, bs, dtype)
    tables = table.view(1, -1).to(DEV)
    sink_dev = sinks.float().to(DEV)
    positions = torch.arange(T, dtype=torch.int32, device=DEV)
    tok_seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    q_dev = q.to(dtype).reshape(T, H * D).to(DEV)
    out = torch.empty(T, H * V, dtype=dtype, device=DEV)
    attend(out, q_dev, kc, vc, positions, tok_seq, tables, [(0, 0, T, 0)], H, G, D, V, scale, 0, cap, sink_dev)
    err = (out.double().cpu() - want).abs().max()
    assert float(err) <= tolerance(dtype, want), f"prompt: {float(err):.3e}"
    # a standing-out far key must matter: without it the last row moves
    if not cap or cap >= 20:  # (a cap of a few units flattens the score that stands out)
        without = plain.attend(qr, torch.cat([kr[:5], kr[6:7], kr[6:]]), vr, scale, cap or None, sinks).reshape(T, H * V)
        assert float((want[699] - without[699]).abs().max()) > 5 * tolerance(dtype, want)
    # single tokens (the decode kernel): the last token, tokens at page borders, the first token
    for p in (699, bs * 9, bs * 9 + 1, bs * 20 - 1, 0, 1):
        one = torch.empty(1, H * V, dtype=dtype, device=DEV)
        attend(one, q_dev[p:p + 1], kc, vc, positions[p:p + 1], tok_seq[:1], tables, [(0, 0, 1, p)], H, G, D,
                         V, scale, 0, cap, sink_dev)
        err = (one.double().cpu()[0] - want[p]).abs().max()
        assert float(err) <= tolerance(dtype, want), f"single token at {p}: {float(err):.3e}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,V,bs", [(4, 2, 64, 64, 16), (3, 3, 24, 40, 16)])
def test_capped_attention_with_sinks_inside_a_window(dtype, H, G, D, V, bs):
    """The mechanisms together with a window (for designs that have one): the key just inside the window
    of the last query and the one just outside it both stand out, and only the first may count."""
    window, T = 100, 300
    gen = torch.Generator().manual_seed(V)
    q = torch.randn(T, H, D, generator=gen, dtype=torch.float64) * 0.5
    k = torch.randn(T, G, D, generator=gen, dtype=torch.float64) * 0.5
    v = torch.randn(T, G, V, generator=gen, dtype=torch.float64)
    direction = torch.randn(D, generator=gen, dtype=torch.float64)
    direction /= direction.norm()
    q[T - 1] = 4.0 * direction
    k[T - window] = 4.0 * direction        # the oldest key the last query sees
    k[T - window - 1] = 6.0 * direction    # one further back: outside
    sinks = torch.linspace(2.0, -2.0, H, dtype=torch.float64)
    scale, cap = 2.0 / math.sqrt(D) * 3, 20.0
    qr, kr, vr = (x.to(dtype).double() for x in (q, k, v))
    want = plain.attend(qr, kr, vr, scale, cap, sinks, window=window).reshape(T, H * V)
    table = scattered_table(-(-T // bs), 2, seed=1)
    kc, vc = fill_cache(k, v, table, bs, dtype, spare=2)
    tables, sink_dev = table.view(1, -1).to(DEV), sinks.float().to(DEV)
    positions = torch.arange(T, dtype=torch.int32, device=DEV)
    tok_seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    q_dev = q.to(dtype).reshape(T, H * D).to(DEV)
    out = torch.empty(T, H * V, dtype=dtype, device=DEV)
    attend(out, q_dev, kc, vc, positions, tok_seq, tables, [(0, 0, T, 0)], H, G, D, V, scale, window, cap, sink_dev)
    assert float((out.double().cpu() - want).abs().max()) <= tolerance(dtype, want)
    one = torch.empty(1, H * V, dtype=dtype, device=DEV)
    attend(one, q_dev[T - 1:], kc, vc, positions[T - 1:], tok_seq[:1], tables, [(0, 0, 1, T - 1)], H, G, D, V, scale,
           window, cap, sink_dev)
    assert float((one.double().cpu()[0] - want[T - 1]).abs().max()) <= tolerance(dtype, want)
    leaked = plain.attend(qr, kr, vr, scale, cap, sinks, window=window + 1).reshape(T, H * V)
    assert float((leaked[T - 1] - want[T - 1]).abs().max()) > 5 * tolerance(dtype, want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,V,rot,interleaved,norm", [(4, 2, 32, 16, 16, True, True), (3, 3, 48, 48, 48, True, True),
                                                            (2, 1, 64, 8, 32, False, True), (5, 1, 24, 40, 0, True, True),
                                                            (2, 2, 16, 16, 8, True, False)])
def test_projection_norm_rotation_and_store(dtype, H, G, D, V, rot, interleaved, norm):
    K = _K()
    T, bs = 90, 16
    gen = torch.Generator().manual_seed(H * 100 + D)
    rows = torch.randn(T, (H + G) * D + G * V, generator=gen, dtype=torch.float64).to(dtype)
    qw = (1.0 + 0.3 * torch.randn(H * D, generator=gen, dtype=torch.float64)).to(dtype)
    kw = (1.0 + 0.3 * torch.randn(G * D, generator=gen, dtype=torch.float64)).to(dtype)
    positions = torch.arange(T) * 3 + 5  # any positions: the pages hold 3 T + 5 tokens
    cfg = {"base": 700.0, "dims": rot, "scaling": {"factor": 3.0, "original": 128, "fast": 8.0, "slow": 1.0}}
    x = rows.double()
    q, k, v = x[:, :H * D], x[:, H * D:(H + G) * D], x[:, (H + G) * D:]
    if norm:
        q, k = plain.rms_norm(q, qw.double(), 1e-5), plain.rms_norm(k, kw.double(), 1e-5)
    q, k = q.reshape(T, H, D), k.reshape(T, G, D)
    mult = 1.0
    if rot:
        if interleaved:
            q, k = plain.rotate_interleaved(q, positions, cfg), plain.rotate_interleaved(k, positions, cfg)
        else:  # pairs (i, i + rot / 2), the same angles
            freq, mult = plain.yarn_frequencies(cfg)
            ang = positions.double()[:, None] * freq[None, :]
            c, s = (torch.cos(ang) * mult)[:, None, :], (torch.sin(ang) * mult)[:, None, :]

            def turn(t):
                out = t.clone()
                a, b = t[..., :rot // 2], t[..., rot // 2:rot]
                out[..., :rot // 2], out[..., rot // 2:rot] = a * c - b * s, b * c + a * s
                return out
            q, k = turn(q), turn(k)
    freq, mult = plain.yarn_frequencies(cfg) if rot else (None, 1.0)
    pages = -(-(3 * T + 5) // bs)
    table = scattered_table(pages, 2, seed=3)
    kc = torch.zeros(pages + 2, G, bs, D, dtype=dtype, device=DEV)
    vc = torch.zeros(pages + 2, G, V, bs, dtype=dtype, device=DEV)
    dev_rows = rows.to(DEV).clone()
    pos_dev = positions.to(torch.int32).to(DEV)
    cos_sin = K.rope_table(pos_dev, freq.float().to(DEV)) if rot else None
    K.qk_norm_rotate_store(dev_rows, H, G, D, V, qw.to(DEV) if norm else None, kw.to(DEV) if norm else None, 1e-5, rot,
                           interleaved, cos_sin, mult, pos_dev, torch.zeros(T, dtype=torch.int32, device=DEV),
                           table.view(1, -1).to(DEV), bs, kc, vc)
    tol = 3e-5 if dtype == torch.float32 else 2e-2
    # angles are formed in float32 on the device (position * float32 frequency): at positions of a few
    # hundred that is 1e-5 radians from the float64 angle
    got_q = dev_rows[:, :H * D].double().cpu().reshape(T, H, D)
    assert float((got_q - q).abs().max()) <= tol * float(q.abs().max())
    kc, vc = kc.cpu(), vc.cpu()
    for t in range(T):
        p = int(positions[t])
        page = int(table[p // bs])
        assert float((kc[page, :, p % bs].double() - k[t]).abs().max()) <= tol * float(k.abs().max())
        assert torch.equal(vc[page, :, :, p % bs].double(), v[t].reshape(G, V))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("G,H,D,V,taps", [(2, 4, 16, 24, 3), (1, 2, 40, 8, 2), (3, 3, 20, 36, 4), (2, 2, 72, 16, 4),
                                          (1, 4, 8, 40, 1), (2, 2, 128, 64, 4)])
def test_delta_rule_with_state_carried_over_steps(dtype, G, H, D, V, taps):
    """Three sequences of unequal length in one step, then the same sequences cut into steps at other
    places (two tokens, one token, a long run), in slots that other sequences used before: the state
    (matrices and the convolutions' last inputs) must carry everything."""
    K = _K()
    gen = torch.Generator().manual_seed(D + 10 * V)
    C = 2 * G * D + H * V
    N = C + H * V + 2 * H
    lengths = (57, 1, 23)
    conv = torch.randn(C, taps, generator=gen, dtype=torch.float64) * 0.5
    a_log = torch.randn(H, generator=gen, dtype=torch.float64) * 0.7
    dt_bias = torch.randn(H, generator=gen, dtype=torch.float64)
    norm_w = (1.0 + 0.3 * torch.randn(V, generator=gen, dtype=torch.float64)).to(dtype)
    projs = [torch.randn(n, N, generator=gen, dtype=torch.float64).to(dtype) for n in lengths]
    # one key direction is written strongly at token 2 of the first sequence and read at its last token:
    # a state that loses early writes shows there
    want = []
    for proj in projs:
        x = proj.double()
        parts = torch.split(x, [G * D, G * D, H * V, H * V, H, H], dim=1)
        want.append(plain.delta_core(*parts, conv[:G * D], conv[G * D:2 * G * D], conv[2 * G * D:], a_log, dt_bias,
                                     norm_w.double(), G, H, D, V, 1e-5))
    slots_total = 5
    state = torch.randn(slots_total, H, V, D, device=DEV)           # what earlier requests left behind
    tail = torch.randn(slots_total, max(taps - 1, 0), C, device=DEV)
    conv_dev, a_dev, dt_dev = conv.float().to(DEV), a_log.float().to(DEV), dt_bias.float().to(DEV)
    tol = 3e-5 if dtype == torch.float32 else 2e-2

    def run(cuts_per_seq, slot_of):
        for s in slot_of:  # a slot is zeroed when a request takes it
            state[s].zero_()
            tail[s].zero_()
        at = [0] * len(lengths)
        got = [[] for _ in lengths]
        step = 0
        while any(a < n for a, n in zip(at, lengths)):
            rows, runs, slots, seqs, positions = [], [], [], [], []
            for i, n in enumerate(lengths):
                if at[i] >= n:
                    continue
                cuts = cuts_per_seq[i]
                c = min(cuts[step % len(cuts)], n - at[i])
                runs += [sum(r.shape[0] for r in rows), c, at[i], 0]
                rows.append(projs[i][at[i]:at[i] + c])
                seqs += [len(slots)] * c
                positions += list(range(at[i], at[i] + c))
                slots.append(slot_of[i])
                got[i].append(c)
                at[i] += c
            proj = torch.cat(rows).to(DEV)
            out = torch.empty(proj.shape[0], H * V, dtype=dtype, device=DEV)
            K.delta_rule_step(proj, out, torch.tensor(seqs, dtype=torch.int32, device=DEV),
                              torch.tensor(positions, dtype=torch.int32, device=DEV),
                              torch.tensor(runs, dtype=torch.int32, device=DEV).view(-1, 4),
                              torch.tensor(slots, dtype=torch.int32, device=DEV), conv_dev, tail, state, a_dev, dt_dev,
                              norm_w.to(DEV), G, H, D, V, taps, 1e-6, 1e-5)
            out = out.double().cpu()
            row = 0
            for i in range(len(lengths)):
                if got[i] and isinstance(got[i][-1], int):
                    c = got[i].pop()
                    got[i].append(out[row:row + c])
                    row += c
            step += 1
        return [torch.cat(g) for g in got]

    for cuts, slot_of in ((((100,), (100,), (100,)), (0, 1, 2)),
                          (((2, 1, 9), (1,), (1, 2)), (3, 0, 4)),
                          (((1,), (1,), (5, 1, 1)), (2, 4, 1))):
        for g, w in zip(run(cuts, slot_of), want):
            assert float((g - w).abs().max()) <= tol * float(w.abs().max())


@pytest.mark.parametrize("dtype", DTYPES)
def test_branch_norm_add_and_activations(dtype):
    K = _K()
    gen = torch.Generator().manual_seed(4)
    T, H = 19, 100
    residual = torch.randn(T, H, generator=gen)
    y = torch.randn(T, H, generator=gen).to(dtype)
    w = (1.0 + 0.2 * torch.randn(H, generator=gen)).to(dtype)
    want = residual.double() + 0.6 * plain.rms_norm(y.double(), w.double(), 1e-5)
    r = residual.to(DEV).clone()
    nxt = torch.empty(T, H, dtype=dtype, device=DEV)
    K.norm_scale_add(r, y.to(DEV), w.to(DEV), 1e-5, 0.6, nxt)
    assert float((r.double().cpu() - want).abs().max()) <= 1e-5
    assert torch.equal(nxt.cpu(), r.cpu().to(dtype))
    # float32 partial sums of a split product are added in order
    parts = torch.randn(3, T, H, generator=gen)
    want = residual.double() + 1.7 * plain.rms_norm(parts.double().sum(0), w.double(), 1e-5)
    r = residual.to(DEV).clone()
    K.norm_scale_add(r, parts.to(DEV), w.to(DEV), 1e-5, 1.7, None)
    assert float((r.double().cpu() - want).abs().max()) <= 1e-5
    x = (torch.randn(T, H, generator=gen) * 3).to(dtype)
    for kind, fn in (("gelu", plain.gelu_erf), ("silu", plain.silu),
                     ("gelu_tanh", lambda z: 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3))))):
        got = x.to(DEV).clone()
        K.activation(got, kind)
        assert float((got.double().cpu() - fn(x.double())).abs().max()) <= (3e-6 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("rows", [1, 8, 16, 40, 64])
@pytest.mark.parametrize("kind", ["gelu", "gelu_tanh", "silu"])
def test_the_few_row_product_with_an_activation_on_its_sums(rows, kind):
    """act(a W^T) for up to 64 rows, the activation on the float32 sums: against the product in float64
    and the plain activation, with one and with several ranges of k."""
    K = _K()
    gen = torch.Generator().manual_seed(rows)
    a = torch.randn(rows, 256, generator=gen).bfloat16()
    w = (torch.randn(328, 256, generator=gen) * 0.2).bfloat16()
    z = a.double() @ w.double().T
    fn = {"gelu": plain.gelu_erf, "silu": plain.silu,
          "gelu_tanh": lambda t: 0.5 * t * (1 + torch.tanh(math.sqrt(2 / math.pi) * (t + 0.044715 * t ** 3)))}[kind]
    want = fn(z)
    for splits in (1, K.whole_sum_splits(328, 256, rows), 2):
        out = torch.empty(rows, 328, dtype=torch.bfloat16, device=DEV)
        K.gemm_skinny_act(out, a.to(DEV), w.to(DEV), kind, splits)
        err = (out.double().cpu() - want).abs().max()
        assert float(err) <= 2.0 ** -8 * float(want.abs().max()), (splits, float(err))
