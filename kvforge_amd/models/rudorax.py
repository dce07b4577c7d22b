"""``Rudorax``: how a Rudorax configuration becomes a list of parts.

A decoder in which every layer is described by itself in ``config.json``.  The stream starts as
the token's embedding times a constant.  A layer is *parallel with two norms*: the mixer reads
one RMS norm of the stream and the feed-forward another (both weights stored around zero), and
their sum goes into the stream.  The mixer is either grouped-query attention (q and k normalised
per head, rotated in neighbouring pairs with YaRN-stretched frequencies, a sliding window, a
sink in the softmax) or a matrix-memory recurrence (mLSTM) with per-request state; the
feed-forward is a layer of routed experts with a shared one.  A stretch of layers may be gone
through several times in a row with the same weights, every pass with cache and state of its
own.  The logits are soft-capped.  Checkpoint names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.mix.{q,k,v,o}``, ``l<i>.mix.{q.norm,k.norm,sink}`` (attention),
``l<i>.mix.{g,norm,i,i.b,f,f.b}`` (mLSTM), ``l<i>.mlp.e<j>.{gate,up,down}``,
``l<i>.mlp.{router,correction}``, ``l<i>.mlp.shared.{gate,up,down}``, ``final.norm``, ``head``.
"""

from __future__ import annotations

from kvforge_amd.config.rudorax import RotaryConfig, RudoraxConfig
from kvforge_amd.parts.base import LayerCall, ModelSpec
from kvforge_amd.parts.embedding import LMHead, TokenEmbedding
from kvforge_amd.parts.positions import YarnStretch
from kvforge_amd.registry import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, part_class,
                                  register_architecture)

ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o"}


def build_rudorax(cfg: RudoraxConfig) -> ModelSpec:
    norm_cls = part_class(NORMS, "rmsnorm_one_plus", "norm")
    attn_cls = part_class(MIXERS, "attention", "mixer")
    mlstm_cls = part_class(MIXERS, "mlstm", "mixer")
    moe_cls = part_class(FEED_FORWARDS, "moe", "feed-forward")
    block_cls = part_class(BLOCKS, "parallel", "block")
    rotary_cls = part_class(POSITIONS, "rotary", "position encoding")
    w, eps = cfg.width, cfg.norm_eps
    rotaries: dict[RotaryConfig, object] = {}    # layers with equal rotations share the tables

    def rotary_of(rot: RotaryConfig | None):
        if rot is None:
            return None
        if rot not in rotaries:
            sc = rot.scaling
            stretch = YarnStretch(sc.factor, sc.original, sc.fast, sc.slow) if sc is not None else None
            rotaries[rot] = rotary_cls(rot.dims, rot.base, stretch, interleaved=True)
        return rotaries[rot]

    blocks = []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}", layer.mixer
        if layer.type == "attention":
            mixer = attn_cls(f"{p}.mix", w, m.heads, m.kv_heads, m.dim, rotary_of(m.rot), scale=m.scale,
                             window=m.window, value_dim=m.vdim, names=ATTENTION_NAMES,
                             qk_norm=("q.norm", "k.norm", eps), sink="sink")
        else:
            mixer = mlstm_cls(f"{p}.mix", w, m.heads, m.dim, m.vdim, m.gate_cap, eps)
        ffn = ffn_norm = None
        if layer.mlp is not None:
            f = layer.mlp
            ffn = moe_cls(f"{p}.mlp", w, f.ff, f.experts, f.top, f.identity, f.shared_ff)
            ffn_norm = norm_cls(f"{p}.norm2", w, eps)
        blocks.append(block_cls(norm_cls(f"{p}.norm1", w, eps), mixer, ffn, w, ffn_norm=ffn_norm))
    # a layer that is gone through again is a further call of the same block: same weights, and
    # (the run order's rule) pages and state slot of its own
    schedule = [LayerCall(i) for i in cfg.run_order()]
    return ModelSpec(config=cfg,
                     embedding=TokenEmbedding("", cfg.vocab_size, w, tensor="embed", scale=cfg.embedding_scale),
                     blocks=blocks, final_norm=norm_cls("final.norm", w, eps),
                     head=LMHead("", cfg.vocab_size, w, tensor="head", softcap=cfg.logit_softcap),
                     positions=list(rotaries.values()), schedule=schedule)


register_architecture(RudoraxConfig.NAME, RudoraxConfig, build_rudorax)
