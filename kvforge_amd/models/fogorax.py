"""``Fogorax``: how a Fogorax configuration becomes a list of parts.

A decoder in which every layer is described by itself in ``config.json``.  The stream starts as
token embedding plus a learned position vector.  A layer is *parallel*: one RMS norm with a single
gain, whose output the mixer (after a token shift) and the dense feed-forward both read; their
sum goes into the stream, and then the layer's own columns of a per-token side table are fed in.
The mixer is attention without rotation under a window with kept first tokens, with an output
gate; a layer may read another layer's keys and values (``kv_from``).  Checkpoint names:
``embed``, ``pos``, ``side.embed``, ``l<i>.norm1``, ``l<i>.shift``, ``l<i>.mix.{q,k,v,g,o}``,
``l<i>.mlp.{gate,up,down}`` with ``.b`` biases, ``l<i>.side.{gate,proj,norm}``, ``final.norm``,
``head``.
"""

from __future__ import annotations

from kvforge_amd.config.fogorax import FogoraxConfig
from kvforge_amd.parts.base import LayerCall, ModelSpec
from kvforge_amd.parts.embedding import LMHead, TokenEmbedding
from kvforge_amd.parts.side import TokenSideInput
from kvforge_amd.registry import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, part_class,
                                  register_architecture)

MIXER_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g"}
MLP_NAMES = {"gate": "gate", "up": "up", "down": "down"}


def build_fogorax(cfg: FogoraxConfig) -> ModelSpec:
    norm_cls = part_class(NORMS, "rmsnorm_scalar", "norm")
    attn_cls = part_class(MIXERS, "attention", "mixer")
    ffn_cls = part_class(FEED_FORWARDS, "gated", "feed-forward")
    block_cls = part_class(BLOCKS, "parallel", "block")
    positions = part_class(POSITIONS, "learned", "position encoding")(
        "pos", cfg.max_position_embeddings, cfg.width)
    w, n = cfg.width, len(cfg.layers)
    blocks, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}", layer.mixer
        mixer = attn_cls(f"{p}.mix", w, m.heads, m.kv_heads, m.dim, None, scale=m.scale,
                         window=m.mask.size, keep_first=m.mask.keep_first, value_dim=m.vdim,
                         gated=True, own_kv=m.kv_from is None, names=MIXER_NAMES)
        ffn = None
        if layer.mlp is not None:
            ffn = ffn_cls(f"{p}.mlp", w, layer.mlp.ff, activation="gelu_tanh", bias=True,
                          names=MLP_NAMES, bias_suffix=".b")
        side = None
        if cfg.side_dim:
            side = TokenSideInput(f"{p}.side", w, cfg.side_dim, cfg.vocab_size, "side.embed",
                                  n * cfg.side_dim, i * cfg.side_dim, cfg.norm_eps)
        blocks.append(block_cls(norm_cls(f"{p}.norm1", w, cfg.norm_eps), mixer, ffn, w,
                                shift_name=f"{p}.shift", after=side))
        # the run order is the layer order, so a layer's place in it is its number
        schedule.append(LayerCall(i, cache_of=m.kv_from))
    return ModelSpec(config=cfg, embedding=TokenEmbedding("", cfg.vocab_size, w, tensor="embed"),
                     blocks=blocks, final_norm=norm_cls("final.norm", w, cfg.norm_eps),
                     head=LMHead("", cfg.vocab_size, w, tensor="head"),
                     positions=[positions], schedule=schedule)


register_architecture(FogoraxConfig.NAME, FogoraxConfig, build_fogorax)
