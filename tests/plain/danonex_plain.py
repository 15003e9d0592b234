"""A plain, slow Danonex decoder: whole sequences, no cache, one function per mechanism.

This module is the oracle the engine's Danonex model is compared with.  It shares no code
with the product package: it does not import it, keeps no pages or state slots, uses no
kernels, and walks every sequence from its first token.  Everything takes a dict of tensors
keyed by checkpoint name and the plain dict of config.json, so the same functions serve any
size.  `dtype` is the working precision (float64 or float32).

The design in this module's own notation (x: residual stream [T, width]; m: residual
multiplier; N_w: RMS norm with weight w, x / sqrt(mean(x^2) + eps) * w):

    x <- E[tokens]
    per layer:   x <- x + m * N_norm1(mixer(x));   if the layer has a feed-forward:
                 x <- x + m * N_norm2(W_down gelu(W_up x))
    logits = logit_scale * E N_final(x)

Mixer "attention": q/k/v projections; one RMS norm over the whole q projection and one over
the whole k projection; interleaved-pair rotation of the first `rot.dims` features of every
head with YaRN-scaled frequencies; scores scale * q.k, soft-capped by c * tanh(s / c); causal
softmax whose denominator also holds exp(sink_h); values summed; output projection.

Mixer "delta": q/k/v projections, each through a causal depthwise convolution over time and
SiLU; q and k made unit vectors per head (q also times dim^-1/2); per head and token a write
strength beta = sigmoid(.) and a decay g = exp(-exp(A_log) * softplus(. + dt_bias)); the
state S [dim, vdim] of a head goes S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;
o = S^T q; o is RMS-normed over vdim, gated by SiLU of a projection and projected out.
"""

from __future__ import annotations

import math

import torch

DELTA_UNIT_EPS = 1e-6  # inside the root when q and k are made unit vectors

# What reduced precision alone does to the logits: with STORAGE set to a type (torch.bfloat16), every
# matrix product reads operands rounded to it and its result is rounded to it, and so are the rotated
# queries and keys, the values, and the activations handed from one product to the next; sums, norms,
# softmax, the recurrence and the residual stay in the working precision.  A test of a reduced-precision
# engine measures its error against the error of this.
STORAGE = None
# (generator, relative size): every product's sums are moved by that much at random before they are
# rounded, as another order of adding moves them (a fraction of a unit in the last place of the
# storage type): two kernels that are both right differ by this, and a model that is touchy
# somewhere (a norm right after a sum that nearly cancels) turns it into visible differences.
JITTER = None


def stored(x: torch.Tensor) -> torch.Tensor:
    return x if STORAGE is None else x.to(STORAGE).to(x.dtype)


def product(h: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    y = stored(h) @ weight.T
    if JITTER is not None:
        y = y * (1.0 + JITTER[1] * torch.randn(y.shape, generator=JITTER[0], dtype=y.dtype))
    return stored(y)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 20.0, z, torch.log1p(torch.exp(torch.clamp(z, max=20.0))))


# --------------------------------------------------------------------------- rotation


def yarn_frequencies(rot: dict, dtype=torch.float64) -> tuple[torch.Tensor, float]:
    """(frequency of every pair [dims / 2], multiplier of cos and sin)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    freq = base ** (-2.0 * i / dims)
    scaling = rot.get("scaling")
    if not scaling:
        return freq.to(dtype), 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    freq = freq / factor * ramp + freq * (1.0 - ramp)
    return freq.to(dtype), 0.1 * math.log(factor) + 1.0


def rotate_interleaved(x: torch.Tensor, positions: torch.Tensor, rot: dict, angle_dtype=None) -> torch.Tensor:
    """x [T, heads, dim]: pairs (2i, 2i+1) of the first rot.dims features turn by position * f_i."""
    dims = int(rot["dims"])
    work = x.dtype
    freq, mult = yarn_frequencies(rot, angle_dtype or work)
    angle = positions.to(freq.dtype)[:, None] * freq[None, :]          # [T, dims/2]
    cos, sin = (torch.cos(angle) * mult).to(work)[:, None, :], (torch.sin(angle) * mult).to(work)[:, None, :]
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


# --------------------------------------------------------------------------- mixers


def attend(q, k, v, scale: float, cap, sinks, positions=None, window=None) -> torch.Tensor:
    """q [T, H, D], k [T, G, D], v [T, G, V], sinks [H] or None -> [T, H, V]; query t sees keys 0..t
    (the design has no window; with one, for other designs that use these kernels, keys t-window+1..t)."""
    T, H = q.shape[0], q.shape[1]
    G, V = k.shape[1], v.shape[2]
    positions = torch.arange(T) if positions is None else positions
    causal = positions[None, :] <= positions[:, None]
    if window:
        causal = causal & (positions[:, None] - positions[None, :] < window)
    out = torch.zeros(T, H, V, dtype=q.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * float(scale)
        if cap:
            s = float(cap) * torch.tanh(s / float(cap))
        s = s.masked_fill(~causal, -math.inf)
        top = s.max(dim=-1, keepdim=True).values
        if sinks is not None:
            top = torch.maximum(top, sinks[head])
        e = torch.exp(s - top)
        denom = e.sum(-1, keepdim=True)
        if sinks is not None:
            denom = denom + torch.exp(sinks[head] - top)
        out[:, head] = (e / denom) @ v[:, g]
    return out


def attention_mixer(h: torch.Tensor, w: dict, prefix: str, mix: dict, eps: float, angle_dtype=None) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, V = int(mix["heads"]), int(mix["kv_heads"]), int(mix["dim"]), int(mix["vdim"])
    q = rms_norm(product(h, w[prefix + "q"]), w[prefix + "q.norm"], eps).view(T, H, D)
    k = rms_norm(product(h, w[prefix + "k"]), w[prefix + "k.norm"], eps).view(T, G, D)
    v = product(h, w[prefix + "v"]).view(T, G, V)
    positions = torch.arange(T)
    if mix.get("rot") and int(mix["rot"].get("dims", 0)):
        q = rotate_interleaved(q, positions, mix["rot"], angle_dtype)
        k = rotate_interleaved(k, positions, mix["rot"], angle_dtype)
    out = attend(stored(q), stored(k), v, mix["scale"], mix.get("softcap"), w[prefix + "sink"])
    return product(out.reshape(T, H * V), w[prefix + "o"])


def causal_conv_silu(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, K]: y[t, c] = silu(sum_j taps[c, j] * x[t - (K - 1 - j), c]), zeros before t = 0."""
    T, C = x.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x)
    for j in range(K):
        y = y + padded[j:j + T] * taps[:, j][None, :]
    return silu(y)


def unit(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt(x.pow(2).sum(-1, keepdim=True) + DELTA_UNIT_EPS)


def delta_recurrence(q, k, v, beta, decay) -> torch.Tensor:
    """q, k [T, G, D] (already unit vectors), v [T, H, V], beta, decay [T, H] -> o [T, H, V].
    Per head:  S <- decay S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q,  S = 0 before the first token."""
    T, G, D = q.shape
    H, V = v.shape[1], v.shape[2]
    out = torch.zeros(T, H, V, dtype=q.dtype)
    for head in range(H):
        g = head // (H // G)
        S = torch.zeros(D, V, dtype=q.dtype)
        for t in range(T):
            S = decay[t, head] * S
            u = beta[t, head] * (v[t, head] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, head] = S.T @ q[t, g]
    return out


def delta_core(qp, kp, vp, gate_p, b_p, a_p, q_conv, k_conv, v_conv, a_log, dt_bias, norm_w, G, H, D, V, eps):
    """Everything of the delta mixer between its input projections and its output projection."""
    T = qp.shape[0]
    q = unit(causal_conv_silu(qp, q_conv).view(T, G, D)) * D ** -0.5
    k = unit(causal_conv_silu(kp, k_conv).view(T, G, D))
    v = causal_conv_silu(vp, v_conv).view(T, H, V)
    beta = torch.sigmoid(b_p)
    decay = torch.exp(-torch.exp(a_log) * softplus(a_p + dt_bias))
    out = delta_recurrence(q, k, v, beta, decay)
    out = out / torch.sqrt(out.pow(2).mean(-1, keepdim=True) + eps) * norm_w * silu(gate_p).view(T, H, V)
    return out.reshape(T, H * V)


def delta_mixer(h: torch.Tensor, w: dict, prefix: str, mix: dict, eps: float) -> torch.Tensor:
    H, G, D, V = int(mix["heads"]), int(mix["kv_heads"]), int(mix["dim"]), int(mix["vdim"])
    out = delta_core(*(product(h, w[prefix + name]) for name in "qkvgba"), w[prefix + "q.conv"], w[prefix + "k.conv"],
                     w[prefix + "v.conv"], w[prefix + "A_log"], w[prefix + "dt_bias"], w[prefix + "norm"], G, H, D, V, eps)
    return product(out, w[prefix + "o"])


def feed_forward(h: torch.Tensor, w: dict, prefix: str) -> torch.Tensor:
    return product(gelu_erf(product(h, w[prefix + "up"])), w[prefix + "down"])


# --------------------------------------------------------------------------- model


def forward(weights: dict, cfg: dict, tokens, dtype=torch.float64, angle_dtype=None, keep_layers: bool = False):
    """Logits [T, vocab] of one sequence (and, with keep_layers, the stream after every layer)."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps, m = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    x = w["embed"][torch.as_tensor(list(tokens), dtype=torch.long)]
    kept = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        if layer["type"] == "attention":
            y = attention_mixer(x, w, p + "mix.", layer["mixer"], eps, angle_dtype)
        elif layer["type"] == "delta":
            y = delta_mixer(x, w, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(f"layer {i}: unknown mixer '{layer['type']}'")
        x = x + m * rms_norm(y, w[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + m * rms_norm(feed_forward(x, w, p + "mlp."), w[p + "norm2"], eps)
        kept.append(x)
    logits = (stored(rms_norm(x, w["final.norm"], eps)) @ w["embed"].T) * float(cfg["logit_scale"])
    return (logits, torch.stack(kept)) if keep_layers else logits


def greedy_generate(weights: dict, cfg: dict, prompt, new_tokens: int, dtype=torch.float64):
    tokens = list(prompt)
    rows = []
    for _ in range(new_tokens):
        logits = forward(weights, cfg, tokens, dtype)[-1]
        rows.append(logits)
        tokens.append(int(torch.argmax(logits)))
    return tokens[len(prompt):], torch.stack(rows)
