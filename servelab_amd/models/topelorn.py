"""Topelorn: a decoder whose config.json lists its layers.

Every layer is a parallel block: with x = LayerNorm(h), h += Mixer(x) + MLP(x)
(one norm, a gain and no bias; the feed-forward may be absent).  The mixer is
one of two attentions over a window (``parts/window_attention.py``); the
feed-forward is the gated one with silu.  The final layer norm is followed by
the embedding table as the output head.  Checkpoint names: ``embed``,
``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.mlp.{gate,up,down}``, ``final.norm``.

Among the layers that mix values, the first keeps its own values for the
others, which mix them into theirs.
"""
from ..config import TopelornConfig, register_architecture
from ..parts.block import ParallelBlock
from ..parts.embedding import OutputHead, TokenEmbedding
from ..parts.feedforward import GatedMLP
from ..parts.model import LayerCall, ModelSpec
from ..parts.norm import LayerNorm
from ..parts.position import RotaryPosition
from ..parts.window_attention import GatedWindowAttention, LatentWindowAttention


def build_topelorn(cfg: TopelornConfig) -> ModelSpec:
    embedding = TokenEmbedding(cfg.vocab, cfg.width, name="embed")
    layers = []
    gave_values = False
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if layer.kind == "attention":
            role = None
            if m.v_mix:
                role = "take" if gave_values else "give"
                gave_values = True
            mixer = GatedWindowAttention(
                cfg.width, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, m.window.size,
                keep_first=m.window.keep_first, norm_eps=cfg.norm_eps, value_mix=role)
        else:
            mixer = LatentWindowAttention(
                cfg.width, m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.scale, m.window.size,
                RotaryPosition(m.rot_dim, m.rot_base, rotary_dim=m.rot_dims), norm_eps=cfg.norm_eps)
        mlp = None
        if layer.mlp is not None:
            mlp = GatedMLP(cfg.width, layer.mlp.ff, names=("gate", "up", "down"))
        block = ParallelBlock(LayerNorm(cfg.width, cfg.norm_eps, name="norm1"), mixer, mlp,
                              names=("", "mix.", "mlp."))
        layers.append((f"l{i}.", block))
    optional = tuple(f"l{i}.mix.vmix" for i, l in enumerate(cfg.layers)
                     if l.kind == "attention" and not l.mixer.v_mix)
    return ModelSpec(
        embedding=("", embedding),
        layers=layers,
        run=[LayerCall(i, i) for i in range(len(cfg.layers))],
        final_norm=("final.", LayerNorm(cfg.width, cfg.norm_eps, name="norm")),
        head=("", OutputHead(cfg.vocab, cfg.width, tied_to=embedding)),
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        eos_token_id=-1,
        optional_tensors=optional,
    )


register_architecture("Topelorn", TopelornConfig.from_hf, build_topelorn, model_type="topelorn")
