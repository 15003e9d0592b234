"""A plain, slow Ritalorn decoder: whole sequences, no cache, one function per mechanism.

This module is the oracle the engine's Ritalorn model is compared with.  It shares no code with
the product package: it does not import it, keeps no pages or state slots, uses no kernels, and
walks every sequence from its first token.  Everything takes a dict of tensors keyed by checkpoint
name and the plain dict of config.json, so the same functions serve any size.  `dtype` is the
working precision (float64 or float32).

The design in this module's own notation (S copies X[s] of the stream, each [T, width]; N_w the
RMS norm x / sqrt(mean(x^2) + eps) * w):

    X[s] <- E[tokens] for every s
    per layer, for the mixer (q = 1) and, if the layer has one, the feed-forward (q = 2):
        u = sum_s in_q[s] X[s];   y = ls_q * sublayer_q(N_norm_q(u))
        X[t] <- sum_s mix_q[s, t] X[s] + out_q[t] y          (every t from the old copies)
    logits = c tanh(H N_final(sum_s X[s]) / c)

Mixer "attention": q, k, v projections with biases; a causal convolution over time on every
channel of each; q and k heads divided by their root mean square (no weight); score
scale * q.k - 2^(-8 (h + 1) / H) (i - j) for the keys j <= i of i's chunk (chunks of mask.size
from position 0); softmax; heads times sigmoid(W_g x); output projection with bias.  A layer with
`kv_from` has only the query side and reads the named layer's keys and values.

Mixer "latent_attention": q projection, heads [dim | rot_dim]; a down projection to kv_rank + rot_dim
features: the first kv_rank RMS-normed with a weight are the latent c, the rest one key part for all
heads; head keys W_uk c, head values W_uv c; rot_dim parts of q and k rotated in pairs (2i, 2i + 1);
score scale * (q_a . k_a + q_b . k_b) over the last mask.size positions; softmax; output projection.

Feed-forward: W_down(gelu_tanh(W_gate x) * (W_up x)).
"""

from __future__ import annotations

import math

import torch

SLOPE_BASE = 8.0

# What reduced precision alone does to the logits: with STORAGE set to a type (torch.bfloat16), every
# matrix product reads operands rounded to it and its result is rounded to it, and so are the queries,
# keys, values and cached latents; sums, norms, softmax and the stream stay in the working precision.
STORAGE = None
# (generator, relative size): every product's sums are moved by that much at random before they are
# rounded, as another order of adding moves them.
JITTER = None


def stored(x: torch.Tensor) -> torch.Tensor:
    return x if STORAGE is None else x.to(STORAGE).to(x.dtype)


def product(h: torch.Tensor, weight: torch.Tensor, bias=None) -> torch.Tensor:
    y = stored(h) @ weight.T
    if bias is not None:
        y = y + bias
    if JITTER is not None:
        y = y * (1.0 + JITTER[1] * torch.randn(y.shape, generator=JITTER[0], dtype=y.dtype))
    return stored(y)


def rms_norm(x: torch.Tensor, weight, eps: float) -> torch.Tensor:
    y = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z.pow(3))))


def causal_conv(u: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """u [T, C], taps [C, n]: y_t = sum_j taps[:, j] * u_(t - n + 1 + j), zeros before the first token."""
    n = taps.shape[1]
    out = torch.zeros_like(u)
    for t in range(u.shape[0]):
        for j in range(n):
            src = t - n + 1 + j
            if src >= 0:
                out[t] += taps[:, j] * u[src]
    return out


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [T, heads, width]: the pairs (2i, 2i + 1), i < dims / 2, turn by position * base^(-2i / dims)."""
    out = x.clone()
    for i in range(dims // 2):
        angle = positions.to(x.dtype) * base ** (-2.0 * i / dims)
        c, s = torch.cos(angle)[:, None], torch.sin(angle)[:, None]
        a, b = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


def distance_slopes(heads: int) -> list:
    return [2.0 ** (-SLOPE_BASE * (h + 1) / heads) for h in range(heads)]


def visible(i: int, j: int, mask: str, size) -> bool:
    """May the query at position i see the key at position j?"""
    if j > i:
        return False
    if not size:
        return True
    if mask == "chunk":
        return i // size == j // size
    return i - j < size


def attend(q, k, v, scale: float, mask: str, size, slope: float = 0.0) -> torch.Tensor:
    """One head: q [T, D], k [T, D], v [T, V] -> [T, V], scores, mask and softmax spelled out."""
    T = q.shape[0]
    out = torch.zeros(T, v.shape[1], dtype=q.dtype)
    for i in range(T):
        keys = [j for j in range(T) if visible(i, j, mask, size)]
        scores = torch.stack([(q[i] * k[j]).sum() * scale - slope * (i - j) for j in keys])
        weights = torch.softmax(scores, dim=0)
        out[i] = (weights[:, None] * v[keys]).sum(0)
    return out


def attend_fast(q, k, v, scale: float, mask: str, size, slope: float = 0.0) -> torch.Tensor:
    """`attend` by matrices (the same numbers; `attend` is the definition and the tests hold the two together)."""
    T = q.shape[0]
    pos = torch.arange(T)
    i, j = pos[:, None], pos[None, :]
    see = j <= i
    if size:
        see = see & ((i // size == j // size) if mask == "chunk" else (i - j < size))
    scores = (q @ k.T) * scale - slope * (i - j).to(q.dtype)
    scores = scores.masked_fill(~see, -math.inf)
    return torch.softmax(scores, dim=-1) @ v


def conv_attention_keys_values(h, w: dict, prefix: str, mix: dict, eps: float):
    """Keys [T, G, D] (convolved, normed) and values [T, G, V] (convolved) of a layer that has its own."""
    T = h.shape[0]
    G, D, V = mix["kv_heads"], mix["dim"], mix["vdim"]
    k = causal_conv(product(h, w[prefix + "k"], w[prefix + "k.b"]), w[prefix + "k.conv"]).view(T, G, D)
    v = causal_conv(product(h, w[prefix + "v"], w[prefix + "v.b"]), w[prefix + "v.conv"]).view(T, G, V)
    return stored(rms_norm(k, None, eps)), stored(v)


def conv_attention_mixer(h, w: dict, prefix: str, mix: dict, eps: float, keys_values, attend_fn=attend_fast):
    T = h.shape[0]
    H, G, D, V = mix["heads"], mix["kv_heads"], mix["dim"], mix["vdim"]
    q = causal_conv(product(h, w[prefix + "q"], w[prefix + "q.b"]), w[prefix + "q.conv"]).view(T, H, D)
    q = stored(rms_norm(q, None, eps))
    k, v = keys_values
    size = (mix.get("mask") or {}).get("size")
    slopes = distance_slopes(H)
    heads = torch.stack([attend_fn(q[:, j], k[:, j // (H // G)], v[:, j // (H // G)], mix["scale"], "chunk", size, slopes[j])
                         for j in range(H)], dim=1)
    gate = torch.sigmoid(product(h, w[prefix + "g"]))
    return product(stored(heads.reshape(T, H * V) * gate), w[prefix + "o"], w[prefix + "o.b"])


def latent_attention_mixer(h, w: dict, prefix: str, mix: dict, eps: float, attend_fn=attend_fast):
    T = h.shape[0]
    H, D, R, V, C = mix["heads"], mix["dim"], mix["rot_dim"], mix["vdim"], mix["kv_rank"]
    positions = torch.arange(T)
    q = product(h, w[prefix + "q"]).view(T, H, D + R)
    down = product(h, w[prefix + "dkv"])
    c = stored(rms_norm(down[:, :C], w[prefix + "dkv.norm"], eps))
    rot = mix.get("rot") or {}
    dims = int(rot.get("dims", 0))
    shared = down[:, C:].reshape(T, 1, R)
    q_rot = q[..., D:]
    if dims:
        shared = rotate_pairs(shared, positions, float(rot["base"]), dims)
        q_rot = rotate_pairs(q_rot, positions, float(rot["base"]), dims)
    shared, q_rot = stored(shared[:, 0]), stored(q_rot)
    k_up = product(c, w[prefix + "uk"]).view(T, H, D)
    values = product(c, w[prefix + "uv"]).view(T, H, V)
    size = (mix.get("mask") or {}).get("size")
    heads = torch.stack([attend_fn(torch.cat([q[:, j, :D], q_rot[:, j]], -1), torch.cat([k_up[:, j], shared], -1),
                                   values[:, j], mix["scale"], "window", size) for j in range(H)], dim=1)
    return product(stored(heads.reshape(T, H * V)), w[prefix + "o"])


def feed_forward(h, w: dict, prefix: str) -> torch.Tensor:
    return product(stored(gelu_tanh(product(h, w[prefix + "gate"])) * product(h, w[prefix + "up"])), w[prefix + "down"])


def hyper_sublayer(X, w: dict, prefix: str, y_of):
    """X [S, T, width]; y_of(u) is the sublayer's scaled output for the read u.  Returns the new copies."""
    S = X.shape[0]
    u = sum(w[prefix + "in"][s] * X[s] for s in range(S))
    y = y_of(u)
    return torch.stack([sum(w[prefix + "mix"][s, t] * X[s] for s in range(S)) + w[prefix + "out"][t] * y for t in range(S)])


def forward(weights: dict, cfg: dict, tokens, dtype=torch.float64, keep_layers: bool = False, attend_fn=attend_fast):
    w = {k: v.to(dtype) for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    X = torch.stack([x.clone() for _ in range(int(cfg["streams"]))])
    kept, layers = {}, []
    for i, layer in enumerate(cfg["layers"]):
        at, mix = f"l{i}.", layer["mixer"]

        def mixer(u, i=i, at=at, mix=mix, layer=layer):
            h = rms_norm(u, w[at + "norm1"], eps)
            if layer["type"] == "latent_attention":
                y = latent_attention_mixer(h, w, at + "mix.", mix, eps, attend_fn)
            else:
                source = mix.get("kv_from")
                if source is None:
                    kept[i] = conv_attention_keys_values(h, w, at + "mix.", mix, eps)
                y = conv_attention_mixer(h, w, at + "mix.", mix, eps, kept[i if source is None else source], attend_fn)
            return w[at + "ls1"] * y

        X = hyper_sublayer(X, w, at + "hc1.", mixer)
        if layer.get("mlp") is not None:
            X = hyper_sublayer(X, w, at + "hc2.", lambda u: w[at + "ls2"] * feed_forward(rms_norm(u, w[at + "norm2"], eps), w, at + "mlp."))
        layers.append(X.sum(0))
    logits = product(rms_norm(X.sum(0), w["final.norm"], eps), w["head"])
    cap = cfg.get("logit_softcap")
    if cap:
        logits = float(cap) * torch.tanh(logits / float(cap))
    return (logits, layers) if keep_layers else logits


def greedy_generate(weights: dict, cfg: dict, prompt, new_tokens: int, dtype=torch.float64):
    """(tokens, the logits each was the argmax of): the whole sequence is run anew for every token."""
    tokens, rows = list(prompt), []
    for _ in range(new_tokens):
        last = forward(weights, cfg, tokens, dtype)[-1]
        rows.append(last)
        tokens.append(int(last.argmax()))
    return tokens[len(prompt):], torch.stack(rows)
