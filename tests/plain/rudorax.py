"""A plain, slow Rudorax decoder: whole sequences, no cache, no carried state, one function per
mechanism, torch on the CPU in 32-bit (or 64-bit, for a truth all but free of rounding).  It is
the oracle the engine's Rudorax model is held to and shares no code with ``kvforge_amd``: it
reads ``config.json`` dictionaries and ``{checkpoint name: tensor}`` dicts itself.

The design in this file's notation (``T`` tokens of one sequence, positions ``0..T-1``):

* stream ``x_t = embed[token_t] * c`` with ``c = embedding.scale``;
* run order: the layers in file order, except that the layers ``loop.start .. loop.stop-1`` are
  gone through ``loop.times`` times in a row (same weights; a pass keeps nothing of another);
* a layer: ``x += mixer(N1(x)) + ff(N2(x))`` with ``N(x) = x / sqrt(mean(x^2) + eps) * (1 + w)``;
* mixer ``attention``: grouped-query softmax attention; q and k are normalised per head
  (``rms * weight``), rotated (neighbouring pairs, the first ``rot.dims`` elements, frequencies
  stretched YaRN-wise), scored with a constant scale under a sliding window; the softmax's
  denominator holds one more term ``exp(sink_h)``;
* mixer ``mlstm``: a matrix memory ``S`` and a normaliser ``n`` per head with exponential input
  gate and sigmoid forget gate in log space, both soft-capped, kept stable by a running maximum;
* feed-forward: routed experts (softmax router, a correction added for the choice only, the
  last few router outputs standing for "pass the input on") plus a shared expert;
* logits ``= cap * tanh(head @ N(x) / cap)``.
"""

from __future__ import annotations

import math

import torch


def stored(x: torch.Tensor, store: torch.dtype | None) -> torch.Tensor:
    """``x`` after a trip through memory in type ``store`` (rounded and widened again), or
    unchanged for ``None``: ``forward(..., store=torch.bfloat16)`` rounds what an engine serving
    in bfloat16 may keep in 16 bits between two operations, and nothing that the design wants
    in 32 bits."""
    return x if store is None else x.to(store).to(x.dtype)


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """``x`` divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def one_plus_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose stored weight lies around zero."""
    return rms(x, eps) * (1.0 + w)


def run_order(config: dict) -> list[int]:
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


# ---------------------------------------------------------------------------------- attention
def yarn_frequencies(dims: int, base: float, scaling: dict | None) -> tuple[torch.Tensor, float]:
    """(frequency of every rotary pair in float64, factor on cos and sin)."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def turns_to_index(t: float) -> float:
        return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(turns_to_index(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turns_to_index(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """``x [T, heads, dim]``: elements ``2i`` and ``2i+1`` (``i < dims/2``) are turned by the
    angle ``position * frequency_i``; the rest of a head passes.  Angles are formed in 32-bit."""
    dims = int(rot["dims"])
    f, mag = yarn_frequencies(dims, float(rot["base"]), rot.get("scaling"))
    a = positions.to(torch.float32)[:, None] * f.to(torch.float32)[None, :]
    cos, sin = (a.cos() * mag).to(x.dtype)[:, None, :], (a.sin() * mag).to(x.dtype)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def window_mask(T: int, size: int) -> torch.Tensor:
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & (i - j < size)


def sink_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                   mask: torch.Tensor, sink: torch.Tensor) -> torch.Tensor:
    """``q [T, H, d]``, ``k [T, G, d]``, ``v [T, G, dv]``, ``sink [H]``.  The weights of a query
    are ``exp(s_j) / (sum_j exp(s_j) + exp(sink_h))``: the sink takes weight and gives nothing."""
    per = q.shape[1] // k.shape[1]
    out = []
    for h in range(q.shape[1]):
        s = (q[:, h] @ k[:, h // per].T) * scale
        s = s.masked_fill(~mask, float("-inf"))
        top = torch.maximum(s.max(-1, keepdim=True).values, sink[h])
        e = torch.exp(s - top)
        p = e / (e.sum(-1, keepdim=True) + torch.exp(sink[h] - top))
        out.append(p @ v[:, h // per])
    return torch.stack(out, dim=1)


def attention_mixer(h: torch.Tensor, w: dict, p: str, m: dict, eps: float,
                    store: torch.dtype | None = None) -> torch.Tensor:
    T = h.shape[0]
    H, d = int(m["heads"]), int(m["dim"])
    G = int(m["kv_heads"]) if m.get("kv_heads") is not None else H
    dv = int(m["vdim"]) if m.get("vdim") is not None else d
    q = stored(h @ w[p + ".q"].T, store).view(T, H, d)
    k = stored(h @ w[p + ".k"].T, store).view(T, G, d)
    v = stored(h @ w[p + ".v"].T, store).view(T, G, dv)
    q, k = rms(q, eps) * w[p + ".q.norm"], rms(k, eps) * w[p + ".k.norm"]
    pos = torch.arange(T)
    if m.get("rot"):
        q, k = rotate(q, pos, m["rot"]), rotate(k, pos, m["rot"])
    q, k = stored(q, store), stored(k, store)
    size = int(m["mask"]["size"]) if m.get("mask") else T
    o = sink_attention(q, k, v, float(m["scale"]), window_mask(T, size), w[p + ".sink"].to(h.dtype))
    return stored(stored(o.reshape(T, H * dv), store) @ w[p + ".o"].T, store)


# ---------------------------------------------------------------------------------- mLSTM
def capped(z: torch.Tensor, cap: float) -> torch.Tensor:
    return cap * torch.tanh(z / cap)


def mlstm_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, li: torch.Tensor,
               lf: torch.Tensor) -> torch.Tensor:
    """One head, token by token.  ``q, k [T, d]`` (q already scaled), ``v [T, dv]``, log input
    gate ``li [T]`` and log forget gate ``lf [T]``.  With ``a = lf_t + m_{t-1}``:
    ``m_t = max(a, li_t)``, ``S_t = e^(a - m_t) S_{t-1} + e^(li_t - m_t) k_t v_t^T``, ``n_t`` the
    same with ``k_t`` alone, ``o_t = S_t^T q_t / (max(|n_t . q_t|, e^(-m_t)) + 1e-6)``.  ``S``,
    ``n`` and ``m`` start at zero."""
    T, d = q.shape
    S = q.new_zeros(d, v.shape[1])
    n = q.new_zeros(d)
    m = q.new_zeros(())
    out = []
    for t in range(T):
        a = lf[t] + m
        m_new = torch.maximum(a, li[t])
        keep, take = torch.exp(a - m_new), torch.exp(li[t] - m_new)
        S = keep * S + take * torch.outer(k[t], v[t])
        n = keep * n + take * k[t]
        m = m_new
        den = torch.maximum((n @ q[t]).abs(), torch.exp(-m)) + 1e-6
        out.append((S.T @ q[t]) / den)
    return torch.stack(out)


def mlstm_mixer(h: torch.Tensor, w: dict, p: str, m: dict, eps: float,
                store: torch.dtype | None = None) -> torch.Tensor:
    T = h.shape[0]
    H, d = int(m["heads"]), int(m["dim"])
    dv = int(m["vdim"]) if m.get("vdim") is not None else d
    cap = float(m["gate_cap"])
    q = stored(h @ w[p + ".q"].T, store).view(T, H, d) * d ** -0.5
    k = stored(h @ w[p + ".k"].T, store).view(T, H, d)
    v = stored(h @ w[p + ".v"].T, store).view(T, H, dv)
    li = capped(h @ w[p + ".i"].T + w[p + ".i.b"], cap)
    lf = torch.nn.functional.logsigmoid(capped(h @ w[p + ".f"].T + w[p + ".f.b"], cap))
    o = torch.stack([mlstm_scan(q[:, j], k[:, j], v[:, j], li[:, j], lf[:, j]) for j in range(H)], dim=1)
    o = rms(o, eps).reshape(T, H * dv) * w[p + ".norm"]
    o = o * torch.sigmoid(stored(h @ w[p + ".g"].T, store))
    return stored(stored(o, store) @ w[p + ".o"].T, store)


# ---------------------------------------------------------------------------------- feed-forward
def expert(h: torch.Tensor, w: dict, p: str, store: torch.dtype | None = None) -> torch.Tensor:
    a = stored(h @ w[p + ".gate"].T, store)
    b = stored(h @ w[p + ".up"].T, store)
    return stored(torch.nn.functional.silu(a) * b, store) @ w[p + ".down"].T


def route(h: torch.Tensor, router: torch.Tensor, correction: torch.Tensor, top: int
          ) -> tuple[torch.Tensor, torch.Tensor]:
    """(chosen outputs of the router ``[T, top]``, their weights ``[T, top]``): chosen by
    probability plus correction, weighted by probability alone, weights summing to one."""
    s = torch.softmax(h @ router.T, dim=-1)
    chosen = torch.topk(s + correction, top, dim=-1).indices
    g = s.gather(-1, chosen)
    return chosen, g / (g.sum(-1, keepdim=True) + 1e-20)


def routed_ff(h: torch.Tensor, w: dict, p: str, mlp: dict, store: torch.dtype | None = None
              ) -> torch.Tensor:
    r = mlp["router"]
    E, top = int(r["experts"]), int(r["top"])
    chosen, weight = route(h, w[p + ".router"], w[p + ".correction"], top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(chosen[t].tolist(), weight[t]):
            y = h[t] if e >= E else stored(expert(h[t:t + 1], w, f"{p}.e{e}", store)[0], store)
            out[t] += g * y
    if mlp.get("shared"):
        out = out + stored(expert(h, w, p + ".shared", store), store)
    return out


# ---------------------------------------------------------------------------------- the model
def forward(config: dict, weights: dict, tokens, dtype: torch.dtype = torch.float32,
            layers_out: list | None = None, store: torch.dtype | None = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one sequence.  ``layers_out``: a list that receives the stream
    after every layer run.  ``store``: see ``stored``."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    tok = torch.as_tensor(tokens, dtype=torch.long)
    eps = float(config["norm"]["eps"])
    x = w["embed"][tok] * float(config["embedding"]["scale"])
    for i in run_order(config):
        layer, p = config["layers"][i], f"l{i}"
        h = stored(one_plus_norm(x, w[p + ".norm1"], eps), store)
        if layer["type"] == "attention":
            delta = attention_mixer(h, w, p + ".mix", layer["mixer"], eps, store)
        elif layer["type"] == "mlstm":
            delta = mlstm_mixer(h, w, p + ".mix", layer["mixer"], eps, store)
        else:
            raise ValueError(f"layer {i}: unknown type {layer['type']!r}")
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "moe":
                raise ValueError(f"layer {i}: unknown feed-forward {layer['mlp']['kind']!r}")
            h2 = stored(one_plus_norm(x, w[p + ".norm2"], eps), store)
            delta = delta + routed_ff(h2, w, p + ".mlp", layer["mlp"], store)
        x = x + delta
        if layers_out is not None:
            layers_out.append(x.clone())
    z = stored(one_plus_norm(x, w["final.norm"], eps), store) @ w["head"].T
    cap = config.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z


def greedy(config: dict, weights: dict, prompt, n: int, dtype: torch.dtype = torch.float32) -> list[int]:
    """``n`` tokens after ``prompt``, each the largest logit of the whole sequence so far."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(config, weights, toks, dtype)[-1].argmax()))
    return toks[len(prompt):]
