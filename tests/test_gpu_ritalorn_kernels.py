"""The kernels behind the Ritalorn parts, each against the plain function of the same mechanism
(tests/plain/ritalorn_plain.py, float64), on inputs made so that a fault shows: a key whose score
stands out just inside and just outside a chunk's or a window's edge, far back among hundreds, and on
both sides of page borders; slopes that matter; gates far from one half; convolutions carried over
steps cut at every place in slots that held other requests' inputs; copies of the stream joined by
matrices with entries of both signs.
"""

import math

import pytest
import torch

from tests.plain import ritalorn_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def _K():
    from paged_attention_engine_amd.kernels import lib
    return lib


def tol(dtype, top):
    return (2e-5 if dtype == torch.float32 else 2.5e-2) * max(top, 1e-3)


def randn(gen, *shape, scale=1.0):
    return torch.randn(*shape, generator=gen, dtype=torch.float64) * scale


# ------------------------------------------------------------------ copies of the stream
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("copies,hidden,parts", [(1, 90, 0), (3, 128, 0), (4, 64, 3), (8, 36, 2)])
def test_joining_reading_and_norming_the_copies(dtype, copies, hidden, parts):
    K = _K()
    gen = torch.Generator().manual_seed(copies * 100 + hidden)
    T, eps = 7, 3e-6
    X = randn(gen, T, copies, hidden, scale=2.0).float()
    mix, outw, inw = randn(gen, copies, copies).float(), randn(gen, copies).float(), randn(gen, copies).float()
    ls, weight = (1 + randn(gen, hidden, scale=0.3)).float(), (1 + randn(gen, hidden, scale=0.3)).float()
    if parts:
        y_parts = randn(gen, parts, T, hidden).float()
        y, y_dev = y_parts.double().sum(0), y_parts.to(DEV)
    else:
        y_dev = randn(gen, T, hidden).to(dtype)
        y, y_dev = y_dev.double(), y_dev.to(DEV)
    w = {"p.in": inw.double(), "p.mix": mix.double(), "p.out": outw.double()}
    # the plain join, then a read with other weights and the norm
    new = plain.hyper_sublayer(X.double().permute(1, 0, 2), w, "p.", lambda u: ls.double() * y)
    read2 = randn(gen, copies).float()
    want = plain.rms_norm(sum(read2[s].double() * new[s] for s in range(copies)), weight.double(), eps)
    streams = X.reshape(T, copies * hidden).contiguous().to(DEV)
    out = torch.empty(T, hidden, dtype=dtype, device=DEV)
    K.hyper_norm(streams, copies, y_dev, ls.to(DEV), mix.to(DEV), outw.to(DEV), read2.to(DEV), weight.to(DEV), eps, out)
    assert float((out.cpu().double() - want).abs().max()) <= tol(dtype, float(want.abs().max()))
    assert float((streams.cpu().double().view(T, copies, hidden).permute(1, 0, 2) - new).abs().max()) <= 1e-5 * float(new.abs().max())
    # some rows only, nothing written back; and a read without anything pending
    before = streams.clone()
    rows = torch.tensor([5, 0, 5, 2], dtype=torch.int32, device=DEV)
    some = torch.empty(4, hidden, dtype=dtype, device=DEV)
    K.hyper_norm(streams, copies, None, None, None, None, read2.to(DEV), weight.to(DEV), eps, some, rows)
    assert torch.equal(streams, before)
    assert float((some.cpu().double() - want[rows.cpu().long()]).abs().max()) <= tol(dtype, float(want.abs().max()))
    assert float((K.hyper_collapse(streams, copies).cpu().double() - new.sum(0)).abs().max()) <= 1e-5 * float(new.abs().max())
    spread = torch.empty(T, copies * hidden, dtype=torch.float32, device=DEV)
    K.hyper_spread(spread, X[:, 0].contiguous().to(DEV), copies)
    assert torch.equal(spread.cpu().view(T, copies, hidden), X[:, :1].expand(T, copies, hidden))


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_gate_with_the_tanh_gelu(dtype):
    K = _K()
    gen = torch.Generator().manual_seed(3)
    x = randn(gen, 5, 2 * 44, scale=2.0).to(dtype)
    want = plain.gelu_tanh(x[:, :44].double()) * x[:, 44:].double()
    out = torch.empty(5, 44, dtype=dtype, device=DEV)
    K.gated_act(out, x.to(DEV), "gelu_tanh")
    assert float((out.cpu().double() - want).abs().max()) <= tol(dtype, float(want.abs().max()))
    assert abs(float(plain.gelu_tanh(torch.tensor(1.0, dtype=torch.float64))) - 0.8411919906082768) < 1e-12


@pytest.mark.parametrize("rows", [1, 8, 40])
def test_the_few_row_gated_product_with_the_tanh_gelu(rows):
    """Gate and up rows alternate in blocks of 8 in the weight; the activation runs on the float32 sums."""
    K = _K()
    gen = torch.Generator().manual_seed(rows)
    inter, hidden = 48, 64
    a = randn(gen, rows, hidden).to(torch.bfloat16)
    gate, up = randn(gen, inter, hidden, scale=0.3).to(torch.bfloat16), randn(gen, inter, hidden, scale=0.3).to(torch.bfloat16)
    w = torch.stack([gate.view(inter // 8, 8, hidden), up.view(inter // 8, 8, hidden)], dim=1).reshape(2 * inter, hidden)
    want = plain.gelu_tanh(a.double() @ gate.double().T) * (a.double() @ up.double().T)
    out = torch.empty(rows, inter, dtype=torch.bfloat16, device=DEV)
    K.gemm_skinny_gated(out, a.to(DEV), w.contiguous().to(DEV), "gelu_tanh")
    assert float((out.cpu().double() - want).abs().max()) <= 1e-2 * float(want.abs().max())


# ------------------------------------------------------------------ convolutions, head norms, cache write
def scattered_table(num_pages: int, spare: int, seed: int):
    gen = torch.Generator().manual_seed(seed)
    return torch.randperm(num_pages + spare, generator=gen)[:num_pages].to(torch.int32)


def runs_tensor(runs):
    return torch.tensor([x for r in runs for x in (r[0], r[1], r[2], 0)], dtype=torch.int32, device=DEV).view(-1, 4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,V,taps,bs", [(4, 2, 16, 24, 3, 16), (3, 3, 40, 8, 4, 8), (2, 1, 22, 18, 1, 16), (5, 0, 32, 32, 2, 16)])
def test_convolution_norm_and_store_whole_and_cut_anywhere(dtype, H, G, D, V, taps, bs):
    """One sequence whole, then the same rows cut into steps of 1, 2, 5, 9 .. tokens in a slot that held
    another request's inputs before (zeroed as the cache manager zeroes a slot that is taken)."""
    K = _K()
    gen = torch.Generator().manual_seed(H * 10 + taps)
    T, eps = 45, 1e-5
    C = H * D + G * (D + V)
    extra = 13  # features behind the convolved ones (a gate's, say) that the kernel must leave alone
    proj = randn(gen, T, C + extra).to(dtype)
    conv = randn(gen, C, taps, scale=0.6).float()
    y = plain.causal_conv(proj[:, :C].double(), conv.double())
    q_want = plain.rms_norm(y[:, :H * D].view(T, H, D), None, eps).reshape(T, H * D)
    k_want = plain.rms_norm(y[:, H * D:H * D + G * D].view(T, G, D), None, eps) if G else None
    v_want = y[:, H * D + G * D:].view(T, G, V) if G else None
    pages = -(-T // bs)
    table = scattered_table(pages, 3, 5)
    tables = torch.stack([torch.zeros(pages, dtype=torch.int32), table]).to(DEV)  # the sequence is row 1
    for cuts in ((T,), (1, 2, 5, 9, 1, 1, 3, 20, 3)):
        kc = torch.zeros(pages + 3, max(G, 1), bs, D, dtype=dtype, device=DEV)
        vc = torch.zeros(pages + 3, max(G, 1), V, bs, dtype=dtype, device=DEV)
        tail = torch.full((3, max(taps - 1, 1), C), 7.0, dtype=torch.float32, device=DEV)  # another request's inputs
        tail[2].zero_()
        q_got = torch.zeros(T, H * D, dtype=dtype)
        at = 0
        for n in cuts:
            rows = proj[at:at + n].to(DEV)
            q_out = torch.empty(n, H * D, dtype=dtype, device=DEV)
            positions = torch.arange(at, at + n, dtype=torch.int32, device=DEV)
            tok_seq = torch.ones(n, dtype=torch.int32, device=DEV)
            runs = runs_tensor([(0, 0, 0), (0, n, at)])
            slots = torch.tensor([0, 2], dtype=torch.int32, device=DEV)
            K.conv_norm_store(rows, q_out, tok_seq, positions, runs, slots, conv.to(DEV), tail[:, :taps - 1] if taps > 1 else None,
                              taps, H, G, D, V, True, eps, tables if G else None, bs, kc if G else None, vc if G else None)
            q_got[at:at + n] = q_out.cpu()
            at += n
        assert at == T
        assert float((q_got.double() - q_want).abs().max()) <= tol(dtype, float(q_want.abs().max())), cuts
        assert float(tail[0].min()) == 7.0 and float(tail[1].min()) == 7.0  # other slots untouched
        if taps > 1:
            assert torch.equal(tail[2, :taps - 1].cpu(), proj[T - taps + 1:, :C].float())
        for t in range(T if G else 0):
            page, off = int(table[t // bs]), t % bs
            assert float((kc[page, :, off].cpu().double() - k_want[t]).abs().max()) <= tol(dtype, float(k_want.abs().max()))
            assert float((vc[page, :, :, off].cpu().double() - v_want[t]).abs().max()) <= tol(dtype, float(v_want.abs().max()))


# ------------------------------------------------------------------ attention with chunks, slopes and a gate
def fill_cache(k, v, table, bs, dtype, spare=3):
    T, G, D = k.shape
    V = v.shape[2]
    pages = table.numel() + spare
    kc = torch.zeros(pages, G, bs, D, dtype=dtype)
    vc = torch.zeros(pages, G, V, bs, dtype=dtype)
    for t in range(T):
        kc[table[t // bs], :, t % bs] = k[t].to(dtype)
        vc[table[t // bs], :, :, t % bs] = v[t].to(dtype)
    return kc.to(DEV), vc.to(DEV)


def stand_out(q, k, v, query: int, key: int, head: int, kv_head: int, size: float):
    """Make key `key` the one that query `query` of head `head` scores far above all others, and its value unlike the rest."""
    k[key, kv_head] = q[query, head] / q[query, head].norm() * size
    v[key, kv_head] = 5.0 + torch.arange(v.shape[2], dtype=v.dtype)


def attend_all_ways(q, kc, vc, table, bs, H, G, D, V, scale, size, chunked, slopes, gate, new_from, dtype):
    """The rows from `new_from` on as the step's tokens (the earlier ones are in the cache already): by the kernel
    that takes any shape, and, where the product would use them, by the matrix-core kernels for runs and for single tokens."""
    K = _K()
    from paged_attention_engine_amd.parts import StepShape
    from paged_attention_engine_amd.parts.attention import attention_work_lists

    T = q.shape[0]
    n = T - new_from
    qd = q[new_from:].reshape(n, H * D).to(dtype).to(DEV)
    gd = gate[new_from:].reshape(n, H * V).to(dtype).to(DEV) if gate is not None else None
    positions = torch.arange(new_from, T, dtype=torch.int32, device=DEV)
    tok_seq = torch.zeros(n, dtype=torch.int32, device=DEV)
    tables = table.view(1, -1).to(DEV)
    sl = None if slopes is None else torch.tensor(slopes, dtype=torch.float32, device=DEV)
    outs = []
    out = torch.empty(n, H * V, dtype=dtype, device=DEV)
    K.paged_attention_masked(out, qd, kc, vc, positions, tok_seq, tables, H, G, D, V, scale, size or 0, chunked, sl, gd)
    outs.append(("any shape", out.cpu().double()))
    if V == D and K.mfma_attention_supported(dtype, H, G, D, bs):
        shape = StepShape((0,), (0,), (n,), (new_from,), bs)
        lists = {name: torch.tensor(flat, dtype=torch.int32, device=DEV).view(-1, width)
                 for name, (flat, width) in attention_work_lists(shape).items()}
        out = torch.zeros(n, H * V, dtype=dtype, device=DEV)
        if n == 1:
            K.attn_decode(out, qd, kc, vc, lists["decode_work"], tables, H, G, D, scale, size or 0, 0.0, None, chunked, sl, gd)
        else:
            K.attn_prefill(out, qd, kc, vc, lists["prefill_tiles"], positions, tables, H, G, D, scale, size or 0, 0.0, None,
                           chunked, sl, gd)
        outs.append(("matrix cores", out.cpu().double()))
    return outs


EDGE_CASES = [
    # H, G, D, V, bs, T, size, chunked: sizes that are and are not multiples of the page, chunks that end at page borders
    (4, 2, 32, 32, 16, 300, 48, True), (4, 2, 32, 32, 16, 300, 50, True), (6, 2, 64, 64, 16, 700, 0, True),
    (3, 1, 24, 40, 8, 130, 20, True), (8, 1, 64, 64, 16, 200, 64, True), (2, 2, 16, 16, 16, 90, 1, True),
    (4, 4, 32, 32, 16, 150, 40, False), (5, 5, 16, 24, 16, 400, 0, False),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,V,bs,T,size,chunked", EDGE_CASES)
@pytest.mark.parametrize("new", ["prompt", "portion", "single"])
def test_keys_at_every_edge_with_slopes_and_gate(dtype, H, G, D, V, bs, T, size, chunked, new):
    """The last query's head 0 scores one key far above the others: in turn the first key it may see, the key just
    before that (which it must not see), a key far back, its own, and keys on both sides of a page border."""
    gen = torch.Generator().manual_seed(T + size)
    scale = 0.3
    slopes = plain.distance_slopes(H)
    last = T - 1
    first_seen = 0 if not size else (last - last % size if chunked else max(0, last - size + 1))
    candidates = {first_seen, max(first_seen - 1, 0), last, max(last - 1, 0), (last // bs) * bs, max((last // bs) * bs - 1, 0),
                  min(first_seen + 1, last), first_seen + (last - first_seen) // 2}
    new_from = {"prompt": 0, "portion": max(T - 37, 0), "single": T - 1}[new]
    for key in sorted(candidates):
        q, k, v = randn(gen, T, H, D), randn(gen, T, G, D), randn(gen, T, G, V)
        gate = randn(gen, T, H, V, scale=2.0)
        # its score is 40 above the rest after the distance bias has been taken off
        stand_out(q, k, v, last, key, 0, 0, (40.0 + slopes[0] * (last - key)) / scale / float(q[last, 0].norm()))
        if dtype == torch.bfloat16:
            q, k, v, gate = (x.to(dtype).double() for x in (q, k, v, gate))
        want = torch.stack([plain.attend_fast(q[:, h], k[:, h // (H // G)], v[:, h // (H // G)], scale,
                                              "chunk" if chunked else "window", size or None, slopes[h]) for h in range(H)], dim=1)
        want = (want * torch.sigmoid(gate)).reshape(T, H * V)[new_from:]
        table = scattered_table(-(-T // bs), 3, T)
        kc, vc = fill_cache(k, v, table, bs, dtype)
        for how, got in attend_all_ways(q, kc, vc, table, bs, H, G, D, V, scale, size, chunked, slopes, gate, new_from, dtype):
            err = float((got - want).abs().max())
            assert err <= tol(dtype, float(want.abs().max())), f"{how}: key {key} of {first_seen}..{last}: {err}"
        # the standing-out key decides the last row's head 0 exactly when it is visible
        seen = plain.visible(last, key, "chunk" if chunked else "window", size or None)
        head0 = want[-1, :V] / torch.sigmoid(gate[last, 0])
        assert (float((head0 - v[key, 0]).abs().max()) < 0.5) == seen


def test_the_spelled_out_attention_and_the_one_by_matrices_agree():
    gen = torch.Generator().manual_seed(1)
    q, k, v = randn(gen, 23, 8), randn(gen, 23, 8), randn(gen, 23, 5)
    for mask, size in (("chunk", 5), ("window", 4), ("window", None), ("chunk", 1)):
        a = plain.attend(q, k, v, 0.7, mask, size, 0.25)
        b = plain.attend_fast(q, k, v, 0.7, mask, size, 0.25)
        assert float((a - b).abs().max()) < 1e-12


# ------------------------------------------------------------------ latent attention
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,R,V,C,dims,bs,T,size", [(3, 16, 8, 24, 40, 8, 16, 150, 20), (2, 24, 16, 8, 16, 8, 8, 100, 7),
                                                      (4, 32, 32, 32, 64, 32, 16, 330, 100), (1, 40, 24, 72, 72, 24, 16, 80, 0),
                                                      (2, 8, 4, 12, 300, 4, 16, 70, 33), (5, 32, 64, 32, 512, 64, 16, 200, 60),
                                                      (20, 16, 32, 16, 64, 32, 32, 90, 0), (12, 16, 32, 16, 128, 32, 16, 75, 17),
                                                      (3, 16, 32, 16, 96, 32, 16, 300, 130), (2, 24, 64, 8, 192, 64, 16, 280, 0),
                                                      (1, 16, 32, 16, 64, 32, 16, 100, 50)])
@pytest.mark.parametrize("new", ["prompt", "portion", "single"])
def test_latent_attention_from_projected_rows_to_heads(dtype, H, D, R, V, C, dims, bs, T, size, new):
    """Projected rows through the latent norm, the rotation, the page write, the fold of the queries, the attention over
    the cached rows and the value product, against the plain mixer's keys and values formed head by head.  One key is made
    to stand out for the last query: the first one its window holds, then the one just outside."""
    K = _K()
    gen = torch.Generator().manual_seed(T + C)
    eps, scale, base = 1e-5, 0.25, 300.0
    mix = {"heads": H, "dim": D, "rot_dim": R, "vdim": V, "kv_rank": C, "scale": scale, "rot": {"base": base, "dims": dims},
           "mask": {"size": size} if size else None}
    w = {"p.q": randn(gen, H * (D + R), 32, scale=0.3), "p.dkv": randn(gen, C + R, 32, scale=0.3),
         "p.dkv.norm": 1 + randn(gen, C, scale=0.2), "p.uk": randn(gen, H * D, C, scale=0.3),
         "p.uv": randn(gen, H * V, C, scale=0.2), "p.o": torch.eye(H * V, dtype=torch.float64)}
    w = {name: t.to(dtype).double() for name, t in w.items()}
    last = T - 1
    first_seen = max(0, last - size + 1) if size else 0
    new_from = {"prompt": 0, "portion": max(T - 37, 0), "single": T - 1}[new]
    for key in sorted({first_seen, max(first_seen - 1, 0), last}):
        h = randn(gen, T, 32).to(dtype).double()
        h[key] = h[key] * 3.0  # a token whose latent and key part are large
        plain.STORAGE = dtype if dtype == torch.bfloat16 else None
        try:
            want = plain.latent_attention_mixer(h, w, "p.", mix, eps)[new_from:]
        finally:
            plain.STORAGE = None
        proj = (h @ torch.cat([w["p.q"], w["p.dkv"]]).T).to(dtype).to(DEV)
        table = scattered_table(-(-T // bs), 2, T)
        latent = torch.zeros(table.numel() + 2, bs, C + R, dtype=dtype, device=DEV)
        positions = torch.arange(T, dtype=torch.int32, device=DEV)
        tok_seq = torch.zeros(T, dtype=torch.int32, device=DEV)
        tables = table.view(1, -1).to(DEV)
        inv_freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float32, device=DEV)
        cos_sin = K.rope_table(positions, inv_freq)
        q_full = torch.zeros(T, H * (C + R), dtype=dtype, device=DEV)
        cores = K.latent_attn_supported(dtype, C + R, C, bs)
        latent_t = torch.zeros(table.numel() + 2, C, bs, dtype=dtype, device=DEV) if cores else None
        K.latent_prepare(proj, q_full, H, D, R, dims, True, C, w["p.dkv.norm"].to(dtype).to(DEV), eps, cos_sin, positions, tok_seq,
                         tables, latent, latent_t)
        up_k_t = w["p.uk"].view(H, D, C).transpose(1, 2).contiguous().to(dtype).to(DEV)
        K.heads_product(q_full.view(T, H, C + R)[:, :, :C], proj[:, :H * (D + R)].view(T, H, D + R)[:, :, :D], up_k_t)
        n = T - new_from
        summed = torch.empty(n, H * C, dtype=dtype, device=DEV)
        K.paged_attention_masked(summed, q_full[new_from:], latent, None, positions[new_from:], tok_seq[new_from:], tables, H, 1,
                                 C + R, C, scale, size or 0)
        heads = torch.empty(n, H * V, dtype=dtype, device=DEV)
        K.heads_product(heads.view(n, H, V), summed.view(n, H, C), w["p.uv"].view(H, V, C).to(dtype).to(DEV))
        if cores:  # the same on the matrix cores: single tokens one column tile, runs two
            from paged_attention_engine_amd.parts import StepShape
            from paged_attention_engine_amd.parts.latent import latent_tiles

            assert torch.equal(latent_t.transpose(1, 2)[table.long()], latent[table.long()][:, :, :C])
            lists = latent_tiles(StepShape((0,), (0,), (n,), (new_from,), bs), K.latent_attn_tokens(H, 1), K.latent_attn_tokens(H, 2))
            fast = torch.zeros(n, H * C, dtype=dtype, device=DEV)
            for name, column_tiles in (("single", 1), ("runs", 2)):
                flat, width = lists[name]
                if flat:
                    tiles = torch.tensor(flat, dtype=torch.int32, device=DEV).view(-1, width)
                    K.latent_attn(fast, q_full[new_from:], latent, latent_t, tiles, column_tiles, positions[new_from:], tables, H, C,
                                  scale, size or 0)
            top = float(summed.float().abs().max())
            assert float((fast.float() - summed.float()).abs().max()) <= 2.5e-2 * top, f"matrix cores, key {key}"
        err = float((heads.cpu().double() - want).abs().max())
        bound = (5e-5 if dtype == torch.float32 else 6e-2) * float(want.abs().max())  # scores of tens: a rounding of q or k is a few 1e-6 of a weight
        assert err <= bound, f"key {key} of {first_seen}..{last}: {err} > {bound}"


def test_rotating_pairs_by_hand():
    """Pair (1, 0) at position 3 with dims 2 turns by 3 radians; features behind `dims` pass unchanged."""
    x = torch.tensor([[[1.0, 0.0, 9.0, 8.0]]], dtype=torch.float64)
    out = plain.rotate_pairs(x, torch.tensor([3]), 10.0, 2)
    assert torch.allclose(out[0, 0], torch.tensor([math.cos(3.0), math.sin(3.0), 9.0, 8.0], dtype=torch.float64))
