"""A plain, slow Fogorax decoder: whole sequences, no cache, no state, one function per
mechanism, torch on the CPU in 32-bit (or 64-bit, for a truth all but free of rounding).  It is
the oracle the engine's Fogorax model is held to and shares no code with ``kvforge_amd``: it
reads ``config.json`` dictionaries and ``{checkpoint name: tensor}`` dicts itself.

The design in this file's notation (``T`` tokens of one sequence, positions ``0..T-1``):

* stream ``x_t = embed[token_t] + pos[t]``;
* every layer: ``h = scalar_rms(x)``, ``x += mixer(shift(h)) + ff(h)``, then the per-layer
  token input ``x += rms(proj @ (gelu(gate @ x) * side[token]))``;
* ``shift(h)_t = h_t + (h_{t-1} - h_t) * mu`` with ``h_{-1} = 0``;
* the mixer is grouped-query softmax attention without rotation under the mask
  ``j <= i and (i - j < size or j < keep_first)``, its heads gated by ``sigmoid(W_g h)``
  before the output projection; a layer with ``kv_from`` takes another layer's keys and values;
* logits are ``head @ scalar_rms(x)``.
"""

from __future__ import annotations

import math

import torch


def stored(x: torch.Tensor, store: torch.dtype | None) -> torch.Tensor:
    """``x`` as it is after a trip through memory in type ``store`` (rounded and widened
    again), or unchanged for ``None``.  ``forward(..., store=torch.bfloat16)`` rounds so every
    tensor that an engine serving in bfloat16 may keep in 16 bits between two operations
    (normalised rows, projections and other products, attention outputs, activations, the
    stream's rows where a product reads them), and nothing else: the stream itself, norms, scores
    and softmax stay as they are.  What that run differs from the
    unrounded one by is the size of rounding alone."""
    return x if store is None else x.to(store).to(x.dtype)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """``x`` divided by its root mean square, eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def scalar_norm(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose gain is one number for all coordinates."""
    return rms(x, eps) * g.reshape(())


def embed(tokens: torch.Tensor, table: torch.Tensor, pos: torch.Tensor) -> torch.Tensor:
    """Token vector plus the learned vector of the token's position (not scaled)."""
    return table[tokens] + pos[: tokens.shape[0]]


def token_shift(h: torch.Tensor, mu: torch.Tensor) -> torch.Tensor:
    """Every token moves towards its predecessor's (unshifted) value by ``mu`` per coordinate;
    the first token's predecessor is zero."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (prev - h) * mu


def window_mask(T: int, size: int, keep_first: int) -> torch.Tensor:
    """``[T, T]`` of booleans: query ``i`` sees key ``j``."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def masked_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                     mask: torch.Tensor) -> torch.Tensor:
    """Softmax attention of ``q [Tq, heads, dim]`` over ``k [Tk, kv_heads, dim]`` and
    ``v [Tk, kv_heads, vdim]``; query head ``h`` uses key/value head ``h // (heads / kv_heads)``;
    ``mask [Tq, Tk]`` says which keys a query sees.  Returns ``[Tq, heads, vdim]``."""
    per = q.shape[1] // k.shape[1]
    out = []
    for h in range(q.shape[1]):
        s = (q[:, h] @ k[:, h // per].T) * scale
        s = s.masked_fill(~mask, float("-inf"))
        out.append(torch.softmax(s, dim=-1) @ v[:, h // per])
    return torch.stack(out, dim=1)


def gated_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gate: torch.Tensor,
                    heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                    mask: torch.Tensor) -> torch.Tensor:
    """``q [T, heads*dim]``, ``k [T, kv_heads*dim]``, ``v [T, kv_heads*vdim]``,
    ``gate [T, heads*vdim]`` (before the sigmoid).  Returns the gated heads side by side."""
    T = q.shape[0]
    o = masked_attention(q.view(T, heads, dim), k.view(T, kv_heads, dim), v.view(T, kv_heads, vdim),
                         scale, mask)
    return o.reshape(T, heads * vdim) * torch.sigmoid(gate)


def dense_ff(h: torch.Tensor, w: dict, p: str, store: torch.dtype | None = None) -> torch.Tensor:
    """``down(gelu(gate h + b) * (up h + b)) + b`` with tensors ``p.gate``, ``p.gate.b`` ..."""
    a = gelu_tanh(stored(h @ w[p + ".gate"].T, store) + w[p + ".gate.b"])
    b = stored(h @ w[p + ".up"].T, store) + w[p + ".up.b"]
    return stored(stored(a * b, store) @ w[p + ".down"].T, store) + w[p + ".down.b"]


def token_side(x: torch.Tensor, side_rows: torch.Tensor, gate: torch.Tensor, proj: torch.Tensor,
               weight: torch.Tensor, eps: float, store: torch.dtype | None = None) -> torch.Tensor:
    """What the per-layer token input adds to the stream ``x``: ``side_rows [T, dim]`` are the
    layer's part of each token's row of the side table."""
    a = stored(stored(x, store) @ gate.T, store)
    y = stored(gelu_tanh(a) * side_rows, store) @ proj.T
    return rms(y, eps) * weight


def forward(config: dict, weights: dict, tokens, dtype: torch.dtype = torch.float32,
            layers_out: list | None = None, store: torch.dtype | None = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one sequence.  ``layers_out``: a list that receives the stream
    after every layer.  ``store``: see ``stored``."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    tok = torch.as_tensor(tokens, dtype=torch.long)
    T = tok.shape[0]
    eps = float(config["norm"]["eps"])
    sdim = int(config["token_side"]["dim"]) if config.get("token_side") else 0
    x = embed(tok, w["embed"], w["pos"])
    kv: dict[int, tuple] = {}
    for i, layer in enumerate(config["layers"]):
        if layer["type"] != "attention":
            raise ValueError(f"layer {i}: unknown type {layer['type']!r}")
        m = layer["mixer"]
        p = f"l{i}"
        h = scalar_norm(x, w[p + ".norm1"], eps)
        hs = stored(token_shift(h, w[p + ".shift"]), store)
        h = stored(h, store)
        H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        if m.get("kv_from") is not None:
            k, v = kv[int(m["kv_from"])]
        else:
            k, v = stored(hs @ w[p + ".mix.k"].T, store), stored(hs @ w[p + ".mix.v"].T, store)
            kv[i] = (k, v)
        mask = window_mask(T, int(m["mask"]["size"]), int(m["mask"]["keep_first"]))
        q, g = stored(hs @ w[p + ".mix.q"].T, store), stored(hs @ w[p + ".mix.g"].T, store)
        if store is None:
            heads = gated_attention(q, k, v, g, H, G, d, dv, float(m["scale"]), mask)
        else:       # the heads make a trip through memory before the gate
            heads = stored(gated_attention(q, k, v, torch.full_like(g, float("inf")), H, G, d, dv,
                                           float(m["scale"]), mask), store)
            heads = stored(heads * torch.sigmoid(g), store)
        delta = stored(heads @ w[p + ".mix.o"].T, store)
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward {layer['mlp']['kind']!r}")
            delta = delta + dense_ff(h, w, p + ".mlp", store)
        x = x + delta
        if sdim:
            x = x + token_side(x, w["side.embed"][tok][:, i * sdim:(i + 1) * sdim],
                               w[p + ".side.gate"], w[p + ".side.proj"], w[p + ".side.norm"], eps, store)
        if layers_out is not None:
            layers_out.append(x.clone())
    return stored(scalar_norm(x, w["final.norm"], eps), store) @ w["head"].T


def greedy(config: dict, weights: dict, prompt, n: int, dtype: torch.dtype = torch.float32) -> list[int]:
    """``n`` tokens after ``prompt``, each the largest logit of the whole sequence so far."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(config, weights, toks, dtype)[-1].argmax()))
    return toks[len(prompt):]
